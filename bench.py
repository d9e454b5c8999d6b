"""Benchmark of the MoE-layer hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload mixtral|fine_grained|large_e] [--no-cpu]

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

WORKLOADS = {
    # name: T, H, I, E, k, routing kind, experts forced empty
    "mixtral": dict(T=16384, H=4096, I=14336, E=8, k=2, kind="uniform", empty=0),
    "fine_grained": dict(T=32768, H=2048, I=1408, E=64, k=8, kind="zipf", empty=4),
    "large_e": dict(T=8192, H=4096, I=1536, E=128, k=8, kind="uniform", empty=0),
}


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=10)
    p.add_argument("--warmup", type=int, default=3)
    p.add_argument("--workload", default="mixtral", choices=list(WORKLOADS))
    p.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    p.add_argument("--no-kernels", action="store_true", help="skip the per-kernel measurements")
    return p.parse_args()


def time_gpu(fn, iters, warmup=2):
    """average milliseconds per call of fn(i), events recorded on the current stream (the launch stream)"""
    import torch

    for i in range(warmup):
        fn(i)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for i in range(iters):
        fn(i)
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / iters


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build runs on one GPU only (got --gpus {args.gpus}); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import fma
    from fma import KernelBackend, MoE, continuous_count, grouped_gemm, swiglu_packed
    from fma.modules.moe import cuda_implementation as ci
    from fma.ops.swiglu.cuda_implementation import swiglu_backward_cuda
    from oracle import moe_oracle as O

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    fma._lib.load()

    c = WORKLOADS[args.workload]
    T, H, I, E, k = c["T"], c["H"], c["I"], c["E"], c["k"]
    R = T * k
    s = 2  # bytes per bf16

    # ---- synthetic inputs (seeded on the CPU generator, then moved: identical bits for every consumer) ----
    g = torch.Generator().manual_seed(42)
    selected, weights = O.make_routing(T, E, k, c["kind"], seed=17, empty_tail=c["empty"])
    x = torch.randn(T, H, generator=g).bfloat16().to(dev)
    dy = torch.randn(T, H, generator=g).bfloat16().to(dev)
    torch.manual_seed(42)
    with torch.device(dev):
        moe = MoE(E, k, H, I, swiglu_packed, True, False, 0.02).to(torch.bfloat16)
    selected_d = selected.to(dev)
    weights_d = weights.bfloat16().to(dev)

    def step():
        moe.zero_grad(set_to_none=True)
        xs = x.detach().requires_grad_()
        ws = weights_d.detach().requires_grad_()
        y = moe._compute_experts(xs, ws, selected_d, KernelBackend.cuda)
        y.backward(dy)
        return y

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    tokens_per_s = T * args.steps / elapsed
    gemm_flops_step = 3 * 2.0 * R * (2 * I * H + I * H)  # fwd + dgrad + wgrad of both projections

    result = {
        "metric": "MoE layer fwd+bwd tokens/s",
        "value": tokens_per_s,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"{args.workload}: MoE layer fwd+bwd, T={T} tokens, hidden={H}, SwiGLU intermediate={I}, "
            f"E={E}, top-k={k}, {c['kind']} routing" + (f", {c['empty']} experts empty" if c["empty"] else ""),
            "router": "excluded (routing computed once, outside the timed region)",
        },
        "layer_gemm_tflops": gemm_flops_step / (ms_per_step * 1e-3) / 1e12,
        "layer_gemm_frac_of_peak": gemm_flops_step / (ms_per_step * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
    }

    # ---- per-kernel measurements -------------------------------------------------------------------------
    if not args.no_kernels:
        kernels = {}
        counts, offsets, perm, eid, inv = ci.build_routing_index(selected_d, E)
        N_fc, K_fc = moe.c_fc.N_array, moe.c_fc.K_array
        N_pj, K_pj = moe.c_proj.N_array, moe.c_proj.K_array
        w1, w2 = moe.c_fc.weight.detach(), moe.c_proj.weight.detach()
        xg = torch.empty(R, H, dtype=torch.bfloat16, device=dev)
        h = torch.empty(R, 2 * I, dtype=torch.bfloat16, device=dev)
        a = torch.empty(R, I, dtype=torch.bfloat16, device=dev)
        o = torch.randn(R, H, device=dev).bfloat16()
        dh = torch.randn(R, 2 * I, device=dev).bfloat16()
        y = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
        d_o = torch.empty(R, H, dtype=torch.bfloat16, device=dev)
        dgates = torch.empty(T, k, dtype=torch.bfloat16, device=dev)
        ci.gather_rows_cuda(x, perm, k, xg)
        iters = max(3, args.steps)

        def mfma(name, flops, ms):
            tf = flops / (ms * 1e-3) / 1e12
            kernels[name] = {"ms": ms, "bound": "mfma", "achieved": tf, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                             "frac": tf / PEAK_BF16_TFLOPS}

        def hbm(name, nbytes, ms):
            gbs = nbytes / (ms * 1e-3) / 1e9
            kernels[name] = {"ms": ms, "bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                             "frac": gbs / PEAK_HBM_GBS, "bytes": nbytes}

        ms = time_gpu(lambda i: ci.grouped_gemm_swiglu_cuda(xg, w1, counts, h, a), iters)
        mfma("up_projection_swiglu_fwd(NT)", 2.0 * R * 2 * I * H, ms)
        ms = time_gpu(lambda i: grouped_gemm(A=a, B=w2, C=None, M_array=counts, N_array=N_pj, K_array=K_pj,
                                             output_shape=(R, H), is_A_transposed=False, is_B_transposed=True), iters)
        mfma("down_projection_fwd(NT)", 2.0 * R * I * H, ms)
        ms = time_gpu(lambda i: grouped_gemm(A=d_o, B=w2, C=None, M_array=counts, N_array=K_pj, K_array=N_pj,
                                             output_shape=(R, I), is_A_transposed=False, is_B_transposed=False), iters)
        mfma("down_projection_dgrad(NN)", 2.0 * R * I * H, ms)
        ms = time_gpu(lambda i: grouped_gemm(A=d_o, B=a, C=None, M_array=N_pj, N_array=K_pj, K_array=counts,
                                             output_shape=(E, H, I), is_A_transposed=True, is_B_transposed=False), iters)
        mfma("down_projection_wgrad(TN)", 2.0 * R * I * H, ms)
        ms = time_gpu(lambda i: grouped_gemm(A=dh, B=w1, C=None, M_array=counts, N_array=K_fc, K_array=N_fc,
                                             output_shape=(R, H), is_A_transposed=False, is_B_transposed=False), iters)
        mfma("up_projection_dgrad(NN)", 2.0 * R * 2 * I * H, ms)
        ms = time_gpu(lambda i: grouped_gemm(A=dh, B=xg, C=None, M_array=N_fc, N_array=K_fc, K_array=counts,
                                             output_shape=(E, 2 * I, H), is_A_transposed=True, is_B_transposed=False), iters)
        mfma("up_projection_wgrad(TN)", 2.0 * R * 2 * I * H, ms)

        # row kernels: algorithmic bytes = each distinct input row once + each output row once + index/gate words
        ms = time_gpu(lambda i: ci.gather_rows_cuda(x, perm, k, xg), 20)
        hbm("gather_rows", T * H * s + R * H * s + R * 4, ms)
        ms = time_gpu(lambda i: ci.combine_cuda(o, inv, weights_d, k, y), 20)
        hbm("combine", R * H * s + R * (4 + s) + T * H * s, ms)
        ms = time_gpu(lambda i: ci.combine_backward_cuda(dy, o, inv, weights_d, k, d_o, dgates), 20)
        hbm("combine_backward", T * H * s + 2 * R * H * s + R * (4 + 2 * s), ms)
        up, gate = h.chunk(2, dim=-1)
        dup, dgate = dh.chunk(2, dim=-1)
        ms = time_gpu(lambda i: swiglu_backward_cuda(gate, up, a, dgate, dup, 1024), 10)
        hbm("swiglu_backward", 5 * R * I * s, ms)
        ms = time_gpu(lambda i: ci.build_routing_index(selected_d, E), 20)
        kernels["build_routing_index(3 launches)"] = {"ms": ms}

        # continuous_count on 16 Mi int32 ids in [0, 64): five distinct 64 MiB buffers (320 MiB > the 256 MiB
        # last-level cache) so that every launch reads from HBM
        for kind in ("uniform", "zipf"):
            ids = [torch.from_numpy(O.make_ids(16 << 20, 64, kind, seed=100 + j)).to(dev) for j in range(5)]
            ms = time_gpu(lambda i: continuous_count(ids[i % 5], 64), 50, warmup=5)
            hbm(f"continuous_count_16Mi_{kind}", (16 << 20) * 4 + 64 * 4, ms)
            del ids
        result["kernels"] = kernels
        dominant = kernels["up_projection_swiglu_fwd(NT)"]
        result["roofline"] = {
            "kernel": "grouped_gemm_kernel<NT, SwiGLU epilogue> (up-projection forward)",
            "bound": "mfma",
            "achieved": dominant["achieved"],
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": dominant["frac"],
            "traffic": None,
        }
        del xg, h, a, o, dh, y, d_o

    # ---- CPU baseline: the oracle (a port of the reference's torch backend) on a bounded sample -------------
    if not args.no_cpu:
        cores = os.cpu_count() or 1
        cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
        torch.set_num_threads(cores)
        T_cpu = max(64, T // 64)
        sel_c, w_c = selected[:T_cpu], weights[:T_cpu].clone().requires_grad_()
        x_c = x[:T_cpu].cpu().float().requires_grad_()
        w1_c = moe.c_fc.weight.detach().cpu().float().requires_grad_()
        w2_c = moe.c_proj.weight.detach().cpu().float().requires_grad_()
        dy_c = dy[:T_cpu].cpu().float()

        def cpu_step():
            for t in (x_c, w_c, w1_c, w2_c):
                t.grad = None
            y_c = O.moe_experts(x_c, w_c, sel_c, w1_c, w2_c)
            y_c.backward(dy_c)

        cpu_step()
        n, t0 = 0, time.perf_counter()
        while n < 3 or (time.perf_counter() - t0 < 10 and n < 50):
            cpu_step()
            n += 1
        cpu_s = (time.perf_counter() - t0) / n
        result["cpu_baseline"] = {
            "value": T_cpu / cpu_s,
            "unit": "tokens/s",
            "cores": cores,
            "kind": "port",
            "sample": f"first {T_cpu} of {T} tokens of the same workload (same H, I, E, k, same routing), fp32 eager "
            f"torch on the host CPU, forward + backward, mean of {n} steps",
        }

    print(json.dumps(result))


if __name__ == "__main__":
    main()
