"""Benchmark of the MoE-layer hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload mixtral|fine_grained|large_e] [--no-cpu]

The headline (metric, value, roofline, kernels) is the Mixtral-shape layer; the same invocation then times the layer step
and the six grouped GEMMs of the other two benchmark shapes and reports them under "workloads".
A step is one forward + backward of the expert path (index construction, gather, up-projection with fused SwiGLU,
down-projection, router-weighted combine, and all their gradients) on synthetic, seeded inputs that are resident in HBM
before the timed region. The router (gate linear, top-k, softmax) is upstream of the path and is not timed. Prints ONE
JSON line: whole-layer tokens/s plus, measured in the same process with events on the launch stream, the duration of
every kernel of the path against its roofline (bf16 MFMA peak for the grouped GEMMs, HBM peak for the row kernels and
continuous_count), and the CPU oracle timed on this machine's host cores on a bounded sample.
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "cute-kernels_amd"))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0  # MI355X HBM3E
PEAK_F32_TFLOPS = 157.3  # MI355X dense fp32 MFMA

WORKLOADS = {
    # name: T, H, I, E, k, routing kind, experts forced empty
    "mixtral": dict(T=16384, H=4096, I=14336, E=8, k=2, kind="uniform", empty=0),
    "fine_grained": dict(T=32768, H=2048, I=1408, E=64, k=8, kind="zipf", empty=4),
    "large_e": dict(T=8192, H=4096, I=1536, E=128, k=8, kind="uniform", empty=0),
}


# Bytes per launch of the up-projection forward kernel crossing the L2 <-> fabric boundary, from two rocprofv3 --pmc runs
# (FETCH_SIZE 7.705e6 KiB, WRITE_SIZE 2.753e6 KiB per dispatch; other pairs of runs read 6.78e6 to 7.55e6 KiB fetched) scaled by what the same counters read for a 1 GiB
# device copy (FETCH_SIZE 0.50, WRITE_SIZE 1.00 of the true bytes); profiles/grouped_gemm_mixtral_counters.txt holds
# the runs. Measured for the mixtral workload only; a constant from those profile runs, not measured by this script.
MEASURED_TRAFFIC_BYTES = {"mixtral": (2 * 7.509e6 + 2.753e6) * 1024}
TRAFFIC_SOURCE = "profiles/grouped_gemm_mixtral_counters.txt (two rocprofv3 --pmc runs of this script; not measured in this run)"


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=10)
    p.add_argument("--warmup", type=int, default=3)
    p.add_argument("--workload", default="mixtral", choices=list(WORKLOADS))
    p.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    p.add_argument("--no-kernels", action="store_true", help="skip the per-kernel measurements")
    p.add_argument("--no-layer", action="store_true", help="skip the whole-layer timing (for short profiler runs)")
    p.add_argument("--fuse-swiglu", type=int, default=-1, choices=[-1, 0, 1],
                   help="1 / 0: compute SwiGLU inside / after the up-projection kernel; -1: the module's default")
    p.add_argument("--permute-experts", action="store_true",
                   help="relabel the experts by a fixed random permutation (skewed routing no longer sorted by expert id)")
    p.add_argument("--zero-operands", action="store_true",
                   help="diagnostic: tokens, weights and gradients all zero in the per-kernel section (same instructions, no "
                        "bits toggling: separates the power limit on the clock from the kernels' schedule)")
    p.add_argument("--only", default="", help="comma-separated substrings: measure only the kernels whose name matches")
    p.add_argument("--no-extra-workloads", action="store_true",
                   help="skip the layer step and GEMMs of the other two benchmark shapes")
    return p.parse_args()


def time_gpu(fn, iters, warmup=3, blocker=None):
    """Median, mean and minimum milliseconds of one launch of fn(i). Every launch is bracketed by its own pair of events on the
    current stream (the stream the kernels are launched on). `blocker` first queues a few milliseconds of other GPU
    work, so that all launches are already in the queue when the GPU reaches them and no host latency is measured."""
    import torch

    for i in range(warmup):
        fn(i)
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(iters)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(iters)]
    torch.cuda.synchronize()
    if blocker is not None:
        blocker()
    for i in range(iters):
        starts[i].record()
        fn(i)
        stops[i].record()
    torch.cuda.synchronize()
    times = sorted(starts[i].elapsed_time(stops[i]) for i in range(iters))
    return times[len(times) // 2], sum(times) / len(times), times[0]


def measure_workload(name, args, full):
    """The layer step of one benchmark shape and the duration of its kernels against their roofs.

    full: every kernel of the path (row kernels, router, norm, bias, index, histogram); otherwise the layer step and the
    grouped GEMMs only. Returns (layer dict, kernels dict, context for the CPU baseline)."""
    import numpy as np
    import torch

    import fma
    from fma import KernelBackend, MoE, swiglu_packed
    from fma.modules.moe import cuda_implementation as ci
    from synthetic_inputs import make_ids, make_routing

    dev = torch.device("cuda", 0)
    c = WORKLOADS[name]
    T, H, I, E, k = c["T"], c["H"], c["I"], c["E"], c["k"]
    R = T * k
    s = 2  # bytes per bf16

    # ---- synthetic inputs (seeded on the CPU generator, then moved: identical bits for every consumer) ----
    g = torch.Generator().manual_seed(42)
    selected, weights = make_routing(T, E, k, c["kind"], seed=17, empty_tail=c["empty"])
    if args.permute_experts:
        selected = torch.randperm(E, generator=torch.Generator().manual_seed(5))[selected]
    x = torch.randn(T, H, generator=g).bfloat16().to(dev)
    dy = torch.randn(T, H, generator=g).bfloat16().to(dev)
    torch.manual_seed(42)
    with torch.device(dev):
        moe = MoE(E, k, H, I, swiglu_packed, True, False, 0.02).to(torch.bfloat16)
    if args.fuse_swiglu >= 0:
        moe.fuse_swiglu = bool(args.fuse_swiglu)
    selected_d = selected.to(dev)
    weights_d = weights.bfloat16().to(dev)

    def step():
        moe.zero_grad(set_to_none=True)
        xs = x.detach().requires_grad_()
        ws = weights_d.detach().requires_grad_()
        y = moe._compute_experts(xs, ws, selected_d, KernelBackend.cuda)
        y.backward(dy)
        return y

    steps, warmup = (0, 0) if args.no_layer else (args.steps, args.warmup)
    if steps:
        # a fresh process on a fresh box runs its first second of steps 5 to 10 % slower (clocks, allocator, page tables):
        # that second is spent here, ahead of the warm-up steps the caller asked for
        t_pre = time.perf_counter()
        while time.perf_counter() - t_pre < 1.0:
            step()
            torch.cuda.synchronize()
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    elapsed = max(time.perf_counter() - t0, 1e-9) if steps else float("inf")
    ms_per_step = elapsed * 1e3 / max(steps, 1)
    tokens_per_s = T * steps / elapsed
    gemm_flops_step = 3 * 2.0 * R * (2 * I * H + I * H)  # fwd + dgrad + wgrad of both projections

    # the same step with the router inside (gate product, top-k, softmax by the fused kernel, and their backward): the
    # expert choice then comes from the randomly initialised gate (close to uniform), not from the workload's routing
    def step_with_router():
        moe.zero_grad(set_to_none=True)
        xs = x.detach().requires_grad_()
        y, _ = moe(xs, kernel_backend=KernelBackend.cuda)
        y.backward(dy)

    ms_with_router = None
    if steps:
        for _ in range(max(1, warmup)):
            step_with_router()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(steps):
            step_with_router()
        torch.cuda.synchronize()
        ms_with_router = (time.perf_counter() - t1) * 1e3 / steps

    # the training step with the choice forced either way: the first projection and its weight gradient gathering their rows
    # through the routing order, or a grouped copy of the tokens written first (ms_per_step above is the layer's own choice)
    ms_step = {}
    if steps:
        for label, gather in (("gather_in_gemm", True), ("grouped_copy", False)):
            moe.gather_in_gemm = gather
            for _ in range(max(1, warmup)):
                step()
            torch.cuda.synchronize()
            t3 = time.perf_counter()
            for _ in range(steps):
                step()
            torch.cuda.synchronize()
            ms_step[label] = (time.perf_counter() - t3) * 1e3 / steps
        moe.gather_in_gemm = None

    # the forward alone with autograd off (evaluation / serving), either way
    ms_forward = {}
    if steps:
        for label, gather in (("gather_in_gemm", True), ("grouped_copy", False)):
            moe.gather_in_gemm = gather
            with torch.no_grad():
                for _ in range(max(1, warmup)):
                    moe._compute_experts(x, weights_d, selected_d, KernelBackend.cuda)
                torch.cuda.synchronize()
                t2 = time.perf_counter()
                for _ in range(steps):
                    moe._compute_experts(x, weights_d, selected_d, KernelBackend.cuda)
                torch.cuda.synchronize()
                ms_forward[label] = (time.perf_counter() - t2) * 1e3 / steps
        moe.gather_in_gemm = None

    layer = {
        "workload": f"{name}: MoE layer fwd+bwd, T={T} tokens, hidden={H}, SwiGLU intermediate={I}, "
        f"E={E}, top-k={k}, {c['kind']} routing" + (f", {c['empty']} experts empty" if c["empty"] else ""),
        "T": T,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": ms_per_step,
        "tokens_per_s": tokens_per_s,
        "ms_per_step_with_router": ms_with_router,
        "tokens_per_s_with_router": None if ms_with_router is None else T / (ms_with_router * 1e-3),
        "ms_per_step_by_row_movement": ms_step or None,
        "ms_forward_no_grad": ms_forward or None,
        "layer_gemm_tflops": gemm_flops_step / (ms_per_step * 1e-3) / 1e12,
        "layer_gemm_frac_of_peak": gemm_flops_step / (ms_per_step * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
    }
    context = dict(x=x, dy=dy, selected=selected, weights=weights, moe=moe, T=T)
    kernels = {}
    if args.no_kernels:
        return layer, kernels, context

    # ---- per-kernel measurements: direct C-ABI calls, one event pair per launch ----------------------------
    lib = fma._lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    BF16 = fma._lib.FMA_BF16
    counts, offsets, perm, eid, inv = ci.build_routing_index(selected_d, E)
    N_pj, K_pj = moe.c_proj.N_array, moe.c_proj.K_array  # (the fp32 GEMM takes the three arrays)
    w1, w2 = moe.c_fc.weight.detach(), moe.c_proj.weight.detach()
    bf = dict(dtype=torch.bfloat16, device=dev)
    xg = torch.empty(R, H, **bf)
    h = torch.empty(R, 2 * I, **bf)
    a = torch.empty(R, I, **bf)
    o = torch.randn(R, H, device=dev).bfloat16()
    dh = torch.randn(R, 2 * I, device=dev).bfloat16()
    y = torch.empty(T, H, **bf)
    d_o = torch.randn(R, H, device=dev).bfloat16()
    da = torch.empty(R, I, **bf)
    dxg = torch.empty(R, H, **bf)
    dw1 = torch.empty(E, 2 * I, H, **bf)
    dw2 = torch.empty(E, H, I, **bf)
    dgates = torch.empty(T, k, **bf)
    if args.zero_operands:
        with torch.no_grad():
            for t in (x, w1, w2, o, dh, d_o):
                t.zero_()
    blk = torch.randn(8192, 8192, device=dev).bfloat16()

    def blocker():  # ~10 ms of queued GPU work, so the host runs ahead of the GPU
        for _ in range(6):
            torch.mm(blk, blk)

    def ok(rc):
        if rc != 0:
            raise RuntimeError(lib.fma_last_error_string().decode())

    VARY_M, VARY_K = fma._lib.FMA_VARY_M, fma._lib.FMA_VARY_K

    def gemm(A, B, D, sizes, vary, m, n, kk, ta, tb):
        # as the layer launches it: one size array (rows per expert) and the two dimensions all experts share by value
        ok(lib.fma_grouped_gemm_ragged(A.data_ptr(), B.data_ptr(), D.data_ptr(), sizes.data_ptr(), None, E, vary, m, n,
                                       kk, ta, tb, 1.0, BF16, stream))

    ok(lib.fma_gather_rows(x.data_ptr(), perm.data_ptr(), R, H, k, xg.data_ptr(), BF16, stream))
    iters = max(20, args.steps)

    only = [w for w in args.only.split(",") if w]

    def want(kernel_name, gemm_kernel=False):
        if not full and not gemm_kernel:
            return False
        return not only or any(w in kernel_name for w in only)

    def mfma(kernel_name, flops, fn, n=iters, nbytes=None, peak=PEAK_BF16_TFLOPS):
        if not want(kernel_name, gemm_kernel=True):
            return
        t = time_gpu(fn, n, warmup=5, blocker=blocker)
        tf = flops / (t[0] * 1e-3) / 1e12
        kernels[kernel_name] = {"ms": t[0], "ms_mean": t[1], "ms_min": t[2], "bound": "mfma", "achieved": tf, "peak": peak,
                                "unit": "TFLOP/s", "frac": tf / peak, "flop": flops}
        if nbytes is not None:  # the second roof: operands read once, output written once
            kernels[kernel_name]["hbm_bytes"] = nbytes
            kernels[kernel_name]["hbm_frac"] = nbytes / (t[0] * 1e-3) / 1e9 / PEAK_HBM_GBS

    def hbm(kernel_name, nbytes, fn, n=50, warmup=10, gemm_kernel=False):
        if not want(kernel_name, gemm_kernel):
            return
        t = time_gpu(fn, n, warmup=warmup, blocker=blocker)
        gbs = nbytes / (t[0] * 1e-3) / 1e9
        kernels[kernel_name] = {"ms": t[0], "ms_mean": t[1], "ms_min": t[2], "bound": "hbm", "achieved": gbs,
                                "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS, "bytes": nbytes}

    w1_b, w2_b = E * 2 * I * H * s, E * H * I * s  # bytes of the two weight tensors
    mfma("up_projection_swiglu_fwd(NT)", 2.0 * R * 2 * I * H,
         lambda i: ok(lib.fma_grouped_gemm_swiglu(xg.data_ptr(), w1.data_ptr(), None, h.data_ptr(), a.data_ptr(),
                                                  counts.data_ptr(), E, I, H, BF16, stream)),
         nbytes=R * H * s + w1_b + R * 3 * I * s)
    # the same launch as a forward without a backward runs it: the pre-activation h is not stored
    mfma("up_projection_swiglu_fwd_inference(NT, h not stored)", 2.0 * R * 2 * I * H,
         lambda i: ok(lib.fma_grouped_gemm_swiglu(xg.data_ptr(), w1.data_ptr(), None, None, a.data_ptr(),
                                                  counts.data_ptr(), E, I, H, BF16, stream)),
         nbytes=R * H * s + w1_b + R * I * s)
    # the same with the gather of the routed rows inside the operand load (x read through perm; no xg), as the layer
    # runs its forward when no backward follows; the flops are the same, the time replaces dispatch_rows + the launch above
    mfma("up_projection_swiglu_fwd_inference_gathered(NT, rows gathered in the operand load)", 2.0 * R * 2 * I * H,
         lambda i: ok(lib.fma_grouped_gemm_gathered(x.data_ptr(), T, perm.data_ptr(), k, w1.data_ptr(), None, None,
                                                    a.data_ptr(), counts.data_ptr(), E, 2 * I, H, 1, BF16, stream)),
         nbytes=T * H * s + R * 4 + w1_b + R * I * s)
    # the unfused pair the fused kernel above replaces (same bits): plain up-projection, then swiglu_forward below
    mfma("up_projection_plain_fwd(NT)", 2.0 * R * 2 * I * H, lambda i: gemm(xg, w1, h, counts, VARY_M, 0, 2 * I, H, 0, 1),
         nbytes=R * H * s + w1_b + R * 2 * I * s)
    mfma("down_projection_fwd(NT)", 2.0 * R * I * H, lambda i: gemm(a, w2, o, counts, VARY_M, 0, H, I, 0, 1),
         nbytes=R * I * s + w2_b + R * H * s)
    mfma("down_projection_dgrad(NN)", 2.0 * R * I * H, lambda i: gemm(d_o, w2, da, counts, VARY_M, 0, I, H, 0, 0),
         nbytes=R * H * s + w2_b + R * I * s)
    # the same product with the backward of SwiGLU in its epilogue (h read, the gradient of h written instead of the
    # gradient of the activation): what the layer's backward runs; it replaces the launch above plus swiglu_backward
    dh_f = torch.empty(R, 2 * I, **bf)
    mfma("down_projection_dgrad_swiglu_bwd(NN + SwiGLU backward)", 2.0 * R * I * H,
         lambda i: ok(lib.fma_grouped_gemm_swiglu_bwd(d_o.data_ptr(), w2.data_ptr(), h.data_ptr(), dh_f.data_ptr(),
                                                      counts.data_ptr(), E, I, H, BF16, stream)),
         nbytes=R * H * s + w2_b + 2 * R * 2 * I * s)
    del dh_f
    mfma("down_projection_wgrad(TN)", 2.0 * R * I * H, lambda i: gemm(d_o, a, dw2, counts, VARY_K, H, I, 0, 1, 0),
         nbytes=R * H * s + R * I * s + w2_b)
    mfma("up_projection_dgrad(NN)", 2.0 * R * 2 * I * H, lambda i: gemm(dh, w1, dxg, counts, VARY_M, 0, H, 2 * I, 0, 0),
         nbytes=R * 2 * I * s + w1_b + R * H * s)
    mfma("up_projection_wgrad(TN)", 2.0 * R * 2 * I * H, lambda i: gemm(dh, xg, dw1, counts, VARY_K, 2 * I, H, 0, 1, 0),
         nbytes=R * 2 * I * s + R * H * s + w1_b)
    # the same product with the gather of the routed rows inside the operand load (x read through perm; no xg): with the
    # gathered forward above, a training step then never writes the grouped copy of the tokens (dispatch_rows below)
    mfma("up_projection_wgrad_gathered(TN, reduction rows gathered in the operand load)", 2.0 * R * 2 * I * H,
         lambda i: ok(lib.fma_grouped_gemm_gathered_wgrad(dh.data_ptr(), x.data_ptr(), T, perm.data_ptr(), k, dw1.data_ptr(),
                                                          counts.data_ptr(), E, 2 * I, H, 1.0, BF16, stream)),
         nbytes=R * 2 * I * s + T * H * s + R * 4 + w1_b)

    # The public op, fma_grouped_gemm (per-group M, N and K arrays in device memory: three launches of which one works), on
    # the shape of the reference's own test (tests/ops/grouped_gemm_test.py:38-52: E=16, N=512, K=4096, sum M = 65536), in
    # the three layouts the layer uses, and the same NT problem through the one-size-array entry point the layer calls
    if full and want("grouped_gemm_op"):
        Mo = [512, 3176, 2048] * 5 + [36856]
        Eo, No, Ko, Ro = len(Mo), 512, 4096, sum(Mo)
        m_o = torch.tensor(Mo, dtype=torch.int32, device=dev).view(torch.uint32)
        n_o, k_o = torch.full_like(m_o, No), torch.full_like(m_o, Ko)
        a_o = torch.randn(Ro * Ko, device=dev).bfloat16()
        b_o = (torch.randn(Eo * No * Ko, device=dev) * 0.02).bfloat16()
        d_o2 = torch.empty(Ro * No, **bf)
        if args.zero_operands:
            a_o.zero_(), b_o.zero_()
        fl_o = 2.0 * Ro * No * Ko
        by_o = (Ro * Ko + Eo * No * Ko + Ro * No) * s
        for lname, ta, tb in (("NT", 0, 1), ("NN", 0, 0), ("TN", 1, 0)):
            mfma(f"grouped_gemm_op({lname}, E=16 N=512 K=4096 sum M=65536, 3 launches)", fl_o,
                 lambda i: ok(lib.fma_grouped_gemm(a_o.data_ptr(), b_o.data_ptr(), d_o2.data_ptr(), m_o.data_ptr(),
                                                   n_o.data_ptr(), k_o.data_ptr(), Eo, ta, tb, 1.0, BF16, stream)),
                 nbytes=by_o)
        mfma("grouped_gemm_op_shape_through_ragged_entry(NT, 1 launch)", fl_o,
             lambda i: ok(lib.fma_grouped_gemm_ragged(a_o.data_ptr(), b_o.data_ptr(), d_o2.data_ptr(), m_o.data_ptr(), None, Eo,
                                                      VARY_M, 0, No, Ko, 0, 1, 1.0, BF16, stream)), nbytes=by_o)
        del a_o, b_o, d_o2

    # the fp32 grouped GEMM (fp32 matrix instruction, 157.3 TFLOP/s peak) on the down-projection's forward shape;
    # only on request (--only fp32): it is not part of the bf16 layer and takes 40 ms per launch
    if only and want("down_projection_fwd_fp32(NT)"):
        a32, w32 = a.float().normal_(), w2.float()
        o32 = torch.empty(R, H, dtype=torch.float32, device=dev)
        mfma("down_projection_fwd_fp32(NT)", 2.0 * R * I * H,
             lambda i: ok(lib.fma_grouped_gemm(a32.data_ptr(), w32.data_ptr(), o32.data_ptr(), counts.data_ptr(),
                                               N_pj.data_ptr(), K_pj.data_ptr(), E, 0, 1, 1.0, fma._lib.FMA_F32,
                                               stream)), n=3, peak=PEAK_F32_TFLOPS)
        del a32, w32, o32

    # the same two forward GEMMs on a batch of a few rows per expert (16 each, e.g. 64 tokens at top-2 of 8): there
    # the kernels are a stream of the expert weights, so the roof is the HBM one and the bytes are the weights' (plus
    # the few activation rows)
    M_dec = max(1, min(64, 128 // E))
    R_dec = M_dec * E
    counts_dec = torch.full((E,), M_dec, dtype=torch.int32, device=dev).view(torch.uint32)
    hbm(f"small_batch_up_fwd(NT + SwiGLU, {M_dec} rows per expert, h not stored)", w1_b + R_dec * (H + I) * s,
        lambda i: ok(lib.fma_grouped_gemm_swiglu(xg.data_ptr(), w1.data_ptr(), None, None, a.data_ptr(),
                                                 counts_dec.data_ptr(), E, I, H, BF16, stream)), n=30, gemm_kernel=True)
    hbm(f"small_batch_down_fwd(NT, {M_dec} rows per expert)", w2_b + R_dec * (H + I) * s,
        lambda i: gemm(a, w2, o, counts_dec, VARY_M, 0, H, I, 0, 1), n=30, gemm_kernel=True)

    # calibration for the profiler's FETCH_SIZE / WRITE_SIZE counters: a plain device copy of known size (ATen's
    # elementwise copy kernel): reads 1 GiB, writes 1 GiB
    if want("hbm_copy_1GiB"):
        src = torch.empty(1 << 29, dtype=torch.bfloat16, device=dev).normal_()
        dst = torch.empty_like(src)
        hbm("hbm_copy_1GiB", 2 * src.numel() * s, lambda i: dst.copy_(src), n=30)
        # what streams of other read : write mixes reach on this part with the runtime's own kernels, for reference beside
        # the row kernels: write only (a fill), and one read for two writes (the mix of gather / dispatch
        # at top-k 2: every input row goes to two output rows)
        hbm("hbm_write_1GiB(fill)", dst.numel() * s, lambda i: dst.fill_(1.0), n=30)
        half = src[: src.numel() // 2]
        hbm("hbm_1read_2writes_1.5GiB(expanded copy)", 3 * half.numel() * s,
            lambda i: dst.view(2, -1).copy_(half.unsqueeze(0).expand(2, -1)), n=30)
        del src, dst, half

    # Row kernels: algorithmic bytes = each distinct input row once + each output row once + index / gate words.
    # Inputs and outputs rotate over several buffer sets whose footprint together exceeds 1 GiB (four times the
    # 256 MiB last-level cache), so that a launch finds neither its inputs nor the lines it writes in that cache.
    def copies(t, set_bytes):
        n = max(2, -(-(1 << 30) // set_bytes))
        return [t] + [t.clone() for _ in range(n - 1)]

    gather_b = T * H * s + R * H * s + R * 4
    combine_b = R * H * s + R * (4 + s) + T * H * s
    combine_bwd_b = T * H * s + 2 * R * H * s + R * (4 + 2 * s)
    if want("gather_rows") or want("dispatch_rows"):
        xs_r, xg_r = copies(x, gather_b), copies(xg, gather_b)
        nr = len(xs_r)
        hbm("gather_rows", gather_b,
            lambda i: ok(lib.fma_gather_rows(xs_r[i % nr].data_ptr(), perm.data_ptr(), R, H, k, xg_r[i % nr].data_ptr(),
                                             BF16, stream)))
        hbm("dispatch_rows", gather_b,
            lambda i: ok(lib.fma_dispatch_rows(xs_r[i % nr].data_ptr(), inv.data_ptr(), T, k, H,
                                               xg_r[i % nr].data_ptr(), BF16, stream)))
        del xs_r, xg_r
    if want("combine"):
        o_r, y_r = copies(o, combine_b), copies(y, combine_b)
        nc = len(o_r)
        hbm("combine", combine_b,
            lambda i: ok(lib.fma_combine(o_r[i % nc].data_ptr(), inv.data_ptr(), weights_d.data_ptr(), T, k, H,
                                         y_r[i % nc].data_ptr(), BF16, stream)))
        dy_r, do_r = copies(dy, combine_bwd_b), copies(d_o, combine_bwd_b)
        nb = len(dy_r)
        hbm("combine_backward", combine_bwd_b,
            lambda i: ok(lib.fma_combine_bwd(dy_r[i % nb].data_ptr(), o_r[i % nc].data_ptr(), inv.data_ptr(),
                                             weights_d.data_ptr(), T, k, H, do_r[i % nb].data_ptr(), dgates.data_ptr(),
                                             BF16, stream)))
        del o_r, y_r, dy_r, do_r
    es = 2 * I  # row stride of the packed pre-activation and of its gradient
    hbm("swiglu_forward", 3 * R * I * s,
        lambda i: ok(lib.fma_swiglu_forward(h.data_ptr() + I * s, h.data_ptr(), a.data_ptr(), R, I, es, es, I, BF16,
                                            stream)), n=30)
    hbm("swiglu_backward", 5 * R * I * s,
        lambda i: ok(lib.fma_swiglu_backward(h.data_ptr() + I * s, h.data_ptr(), da.data_ptr(), dh.data_ptr() + I * s,
                                             dh.data_ptr(), R, I, es, es, I, es, es, BF16, stream)), n=30)
    # router: x and the gate weight read once, logits / weights / choice / histogram written. Three copies of x
    # (together larger than the 256 MiB last-level cache) are rotated so that every launch reads from HBM.
    if want("router"):
        wg = moe.gate.weight.detach()
        xs3 = [x] + [x.clone() for _ in range(2)]
        lg = torch.empty(T, E, **bf)
        rw = torch.empty(T, k, **bf)
        sel32 = torch.empty(T, k, dtype=torch.int32, device=dev)
        cnt = torch.empty(E, dtype=torch.uint32, device=dev)
        tbh = torch.empty((T + 15) // 16, E, dtype=torch.uint32, device=dev)
        # as the MoE module calls it: with the histogram per block of 16 tokens that the index build starts from
        hbm("router_topk", T * H * s + E * H * s + T * E * s + T * k * (s + 4) + tbh.numel() * 4,
            lambda i: ok(lib.fma_router_topk(xs3[i % 3].data_ptr(), wg.data_ptr(), T, H, E, k, lg.data_ptr(),
                                             rw.data_ptr(), sel32.data_ptr(), None, tbh.data_ptr(), BF16, stream)))
        assert int(tbh.view(torch.int32).sum()) == T * k, "router block histogram does not sum to T * top_k"
        ok(lib.fma_router_topk(x.data_ptr(), wg.data_ptr(), T, H, E, k, lg.data_ptr(), rw.data_ptr(),
                               sel32.data_ptr(), cnt.data_ptr(), None, BF16, stream))
        assert int(cnt.view(torch.int32).sum()) == T * k, "router histogram does not sum to T * top_k"

        def aten_router(i):  # the same results from library calls: gate linear, top-k, fp32 softmax, cast
            logits = torch.nn.functional.linear(xs3[i % 3], wg)
            values, _ = logits.topk(k, dim=-1)
            torch.softmax(values.float(), dim=-1).to(torch.bfloat16)

        t = time_gpu(aten_router, 20, blocker=blocker)
        kernels["router_aten(linear+topk+softmax, 4+ launches)"] = {"ms": t[0], "ms_mean": t[1]}
        dlg = torch.randn(T, E, device=dev).bfloat16()
        drw = torch.randn(T, k, device=dev).bfloat16()
        dlg_out = torch.empty(T, E, **bf)
        # a few MB at most: bound by launch latency, so only the time is reported
        t = time_gpu(lambda i: ok(lib.fma_router_topk_bwd(lg.data_ptr(), sel32.data_ptr(), drw.data_ptr(),
                                                          dlg.data_ptr(), T, E, k, dlg_out.data_ptr(), BF16, stream)),
                     20, blocker=blocker)
        kernels["router_topk_backward"] = {"ms": t[0], "ms_mean": t[1], "bytes": 3 * T * E * s + T * k * (s + 4)}
        del xs3
    # residual add + RMSNorm on the layer's residual stream [T, H]: forward reads x and the residual and writes the
    # normalised activations and the new residual; backward reads the saved residual and both incoming gradients and
    # writes the two input gradients (plus the per-workgroup partial weight gradients and their sum)
    if want("rmsnorm"):
        fwd_b, bwd_b = 4 * T * H * s + H * s + T * 4, 5 * T * H * s + H * (s + 4) + T * 4
        nw = (1 + 0.1 * torch.randn(H, device=dev)).bfloat16()
        nn_ = max(2, -(-(1 << 30) // fwd_b))  # buffer sets, rotated like the row kernels' above
        x_n = [x] + [x.clone() for _ in range(nn_ - 1)]
        res_in = [torch.randn(T, H, device=dev).bfloat16() for _ in range(nn_)]
        n_out = [torch.empty(T, H, **bf) for _ in range(nn_)]
        n_added = [torch.empty(T, H, **bf) for _ in range(nn_)]
        n_inv = torch.empty(T, dtype=torch.float32, device=dev)
        hbm("fused_residual_add_rmsnorm_fwd", fwd_b,
            lambda i: ok(lib.fma_fused_residual_add_rmsnorm_fwd(x_n[i % nn_].data_ptr(), res_in[i % nn_].data_ptr(),
                                                                nw.data_ptr(), n_out[i % nn_].data_ptr(),
                                                                n_added[i % nn_].data_ptr(), n_inv.data_ptr(), T, H,
                                                                1e-5, 1.0, BF16, stream)))
        ws_n = torch.empty(max(lib.fma_fused_residual_add_rmsnorm_bwd_workspace_bytes(T, H), 4), dtype=torch.uint8,
                           device=dev)
        n_dw = torch.empty(H, dtype=torch.float32, device=dev)
        # the forward's buffers serve as the backward's: saved residual, two incoming gradients, two outputs
        hbm("fused_residual_add_rmsnorm_bwd(2 launches)", bwd_b,
            lambda i: ok(lib.fma_fused_residual_add_rmsnorm_bwd(n_added[i % nn_].data_ptr(), nw.data_ptr(),
                                                                x_n[i % nn_].data_ptr(), res_in[i % nn_].data_ptr(),
                                                                n_inv.data_ptr(), n_out[(i + 1) % nn_].data_ptr(),
                                                                n_added[(i + 1) % nn_].data_ptr(), n_dw.data_ptr(), T,
                                                                H, 1e-5, 1.0, ws_n.data_ptr(), ws_n.numel(), BF16,
                                                                stream)))
        del x_n, res_in, n_out, n_added, ws_n
    # per-expert bias on the up-projection's output [R, 2I] (layers built with add_bias=True)
    if want("expert_bias"):
        b1 = torch.randn(E, 2 * I, device=dev).bfloat16()
        db1 = torch.empty(E, 2 * I, **bf)
        ws_b = torch.empty(max(lib.fma_expert_bias_grad_workspace_bytes(E, R, 2 * I), 4), dtype=torch.uint8,
                           device=dev)
        hbm("expert_bias_add", 2 * R * 2 * I * s + E * 2 * I * s,
            lambda i: ok(lib.fma_expert_bias_add(h.data_ptr(), b1.data_ptr(), counts.data_ptr(), E, R, 2 * I, BF16,
                                                 stream)), n=30)
        hbm("expert_bias_grad(2 launches)", R * 2 * I * s + E * 2 * I * s,
            lambda i: ok(lib.fma_expert_bias_grad(dh.data_ptr(), counts.data_ptr(), E, R, 2 * I, db1.data_ptr(),
                                                  ws_b.data_ptr(), ws_b.numel(), BF16, stream)), n=30)
    if want("build_routing_index"):
        ws_idx = torch.empty(max(lib.fma_moe_build_index_workspace_bytes(R, E), 4) // 4, dtype=torch.int32, device=dev)
        t = time_gpu(lambda i: ok(lib.fma_moe_build_index(selected_d.data_ptr(), 8, R, E, counts.data_ptr(),
                                                          offsets.data_ptr(), perm.data_ptr(), eid.data_ptr(),
                                                          inv.data_ptr(), ws_idx.data_ptr(), ws_idx.numel() * 4, stream)),
                     20, blocker=blocker)
        kernels["build_routing_index(3 launches)"] = {"ms": t[0], "ms_mean": t[1]}
        # as the layer runs it behind the fused router: int32 choices and their histogram per block of 16 tokens (here
        # made with torch; the call overwrites it, so every launch gets a copy of its own)
        ids32 = selected_d.reshape(-1).to(torch.int32)
        key = (torch.arange(R, device=dev) // (16 * k)) * E + ids32
        hist0 = torch.bincount(key, minlength=((T + 15) // 16) * E).to(torch.int32)
        n_idx = 20
        hists = [hist0.clone() for _ in range(n_idx + 3)]
        calls = iter(range(n_idx + 3))
        want_perm = perm.clone()
        t = time_gpu(lambda i: ok(lib.fma_moe_build_index_from_hist(ids32.data_ptr(), R, E, k, hists[next(calls)].data_ptr(),
                                                                    counts.data_ptr(), offsets.data_ptr(), perm.data_ptr(),
                                                                    eid.data_ptr(), inv.data_ptr(), stream)),
                     n_idx, blocker=blocker)
        assert torch.equal(perm, want_perm), "index build from the router's histogram differs"
        kernels["build_routing_index_from_router_histogram(2 launches)"] = {"ms": t[0], "ms_mean": t[1]}
        del hists

    # continuous_count on 16 Mi int32 ids in [0, 64): five distinct 64 MiB buffers (320 MiB > the 256 MiB
    # last-level cache) so that every launch reads from HBM. The figure covers both launches of one call
    # (count + reduce).
    n_ids, bins = 16 << 20, 64
    for kind in ("uniform", "zipf"):
        if not want(f"continuous_count_16Mi_{kind}"):
            continue
        ws_cnt = torch.empty(lib.fma_continuous_count_workspace_bytes(n_ids, bins), dtype=torch.uint8, device=dev)
        out_cnt = torch.empty(bins, dtype=torch.uint32, device=dev)
        ids = [torch.from_numpy(make_ids(n_ids, bins, kind, seed=100 + j)).to(dev) for j in range(5)]
        hbm(f"continuous_count_16Mi_{kind}", n_ids * 4 + bins * 4,
            lambda i: ok(lib.fma_continuous_count(ids[i % 5].data_ptr(), 4, n_ids, out_cnt.data_ptr(), bins,
                                                  ws_cnt.data_ptr(), ws_cnt.numel(), stream)), n=50, warmup=5)
        expect = np.bincount(make_ids(n_ids, bins, kind, seed=100 + 49 % 5), minlength=bins)
        assert np.array_equal(out_cnt.cpu().view(torch.int32).numpy().astype(np.int64), expect), "count mismatch"
        del ids
    # The same histogram over 256 Mi ids (1 GiB per launch, two buffers rotated): the launch's fixed cost (second launch,
    # ramp-up) is then a few percent of the time and the figure is the rate the count kernel streams at.
    if want("continuous_count_256Mi_uniform"):
        n_big = 256 << 20
        ws_big = torch.empty(lib.fma_continuous_count_workspace_bytes(n_big, bins), dtype=torch.uint8, device=dev)
        out_big = torch.empty(bins, dtype=torch.uint32, device=dev)
        big = [torch.randint(0, bins, (n_big,), dtype=torch.int32, device=dev) for _ in range(2)]
        hbm("continuous_count_256Mi_uniform", n_big * 4 + bins * 4,
            lambda i: ok(lib.fma_continuous_count(big[i % 2].data_ptr(), 4, n_big, out_big.data_ptr(), bins,
                                                  ws_big.data_ptr(), ws_big.numel(), stream)), n=20, warmup=3)
        expect_big = torch.bincount(big[19 % 2], minlength=bins)
        assert torch.equal(out_big.view(torch.int32).long(), expect_big), "count mismatch (256 Mi ids)"
        del big, ws_big
    return layer, kernels, context


def cpu_baseline(context, name):
    """The oracle (a port of the reference's torch backend) on the host cores, on a bounded sample of the workload."""
    import numpy as np
    import torch

    from oracle import moe_oracle as O
    from synthetic_inputs import make_ids

    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    x, dy, selected, weights, moe, T = (context[key] for key in ("x", "dy", "selected", "weights", "moe", "T"))

    def progress(msg):  # keeps a watchdog that looks for output quiet during the CPU leg
        print(f"bench.py: cpu baseline: {msg}", file=sys.stderr, flush=True)

    # One fixed configuration whatever the host's speed, so that the figure compares between runs: bf16, the first T/16
    # tokens, one warm-up step and three timed ones (about 2 s per step on the hosts measured).
    dtype, T_cpu, n = torch.bfloat16, max(64, T // 16), 3
    sel_c, w_c = selected[:T_cpu], weights[:T_cpu].to(dtype).requires_grad_()
    x_c = x[:T_cpu].cpu().to(dtype).requires_grad_()
    w1_c = moe.c_fc.weight.detach().cpu().to(dtype).requires_grad_()
    w2_c = moe.c_proj.weight.detach().cpu().to(dtype).requires_grad_()
    dy_c = dy[:T_cpu].cpu().to(dtype)

    def cpu_step():
        for t in (x_c, w_c, w1_c, w2_c):
            t.grad = None
        O.moe_experts(x_c, w_c, sel_c, w1_c, w2_c).backward(dy_c)

    progress(f"{dtype}, {T_cpu} tokens on {cores} threads, warm-up step")
    cpu_step()
    t0 = time.perf_counter()
    for i in range(n):
        cpu_step()
        progress(f"step {i + 1} of {n}, {time.perf_counter() - t0:.1f} s")
    wall = time.perf_counter() - t0
    cpu_s = wall / n
    out = {
        "value": T_cpu / cpu_s,
        "unit": "tokens/s",
        "cores": cores,
        "kind": "port",
        "sample": f"first {T_cpu} of {T} tokens of the {name} workload (same H, I, E, k, same routing), {dtype} eager torch on "
        f"the host CPU, forward + backward, mean of {n} steps after one warm-up step ({wall:.1f} s of wall time). Not linear "
        "in the token count: the weight-gradient pass writes (and the step then zeroes) the full-size expert weights whatever "
        "the number of tokens.",
    }
    # continuous_count beside it: torch.bincount, the routine the reference's torch backend calls
    # (fma/ops/continuous_count/__init__.py:36), on the same 16 Mi int32 ids on the host
    ids_c = torch.from_numpy(make_ids(16 << 20, 64, "uniform", seed=100))
    expect = np.bincount(ids_c.numpy(), minlength=64)
    assert np.array_equal(O.continuous_count(ids_c.numpy()[: 1 << 16], 64), np.bincount(ids_c.numpy()[: 1 << 16], minlength=64))
    got = torch.bincount(ids_c, minlength=64)
    assert np.array_equal(got.numpy(), expect)
    t0 = time.perf_counter()
    for _ in range(5):
        torch.bincount(ids_c, minlength=64)
    cnt_s = (time.perf_counter() - t0) / 5
    out["continuous_count_16Mi"] = {"ms": cnt_s * 1e3, "GB/s": ids_c.numel() * 4 / cnt_s / 1e9, "cores": torch.get_num_threads(),
                                    "routine": "torch.bincount on int32 ids (ATen's CPU histogram), threads available to torch as stated"}
    return out


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build runs on one GPU only (got --gpus {args.gpus}); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    import fma

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(torch.device("cuda", 0))
    fma._lib.load()

    layer, kernels, context = measure_workload(args.workload, args, full=True)
    result = {
        "metric": "MoE layer fwd+bwd tokens/s",
        "value": layer["tokens_per_s"],
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": layer["steps"],
        "warmup": layer["warmup"],
        "ms_per_step": layer["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": layer["workload"],
            "router": "excluded (routing computed once, outside the timed region); ms_per_step_with_router includes it",
        },
        "ms_per_step_with_router": layer["ms_per_step_with_router"],
        "ms_per_step_by_row_movement": layer["ms_per_step_by_row_movement"],
        "ms_forward_no_grad": layer["ms_forward_no_grad"],
        "tokens_per_s_with_router": layer["tokens_per_s_with_router"],
        "layer_gemm_tflops": layer["layer_gemm_tflops"],
        "layer_gemm_frac_of_peak": layer["layer_gemm_frac_of_peak"],
    }
    if kernels:
        result["kernels"] = kernels
        dominant = kernels.get("up_projection_swiglu_fwd(NT)") or next(iter(kernels.values()))
        result["roofline"] = {
            "kernel": "ragged_gemm_kernel<NT, SwiGLU epilogue> (up-projection forward)",
            "bound": "mfma",
            "achieved": dominant["achieved"],
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": dominant["frac"],
            "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload),
            "traffic_source": TRAFFIC_SOURCE if args.workload in MEASURED_TRAFFIC_BYTES else None,
        }

    # ---- CPU baseline on the headline workload, before its tensors are released ----
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(context, args.workload)
    del context, layer, kernels
    torch.cuda.empty_cache()

    # ---- the other two benchmark shapes: layer step and grouped GEMMs ----
    extra = [] if (args.no_extra_workloads or args.only or args.no_layer or args.workload != "mixtral") else ["fine_grained", "large_e"]
    if extra:
        result["workloads"] = {}
    for name in extra:
        layer, kernels, context = measure_workload(name, args, full=False)
        del context
        entry = {key: layer[key] for key in ("workload", "ms_per_step", "tokens_per_s", "ms_per_step_with_router",
                                             "ms_per_step_by_row_movement", "ms_forward_no_grad", "layer_gemm_tflops", "layer_gemm_frac_of_peak")}
        entry["kernels"] = kernels
        result["workloads"][name] = entry
        torch.cuda.empty_cache()

    print(json.dumps(result))


if __name__ == "__main__":
    main()
