"""GPU parity of the fused router (fma_router_topk / fma_router_topk_bwd through the custom ops) against the oracle.

What can be exact is checked exactly: the expert choice is a function of the logits the kernel itself returns, so it
is compared with the oracle's top-k of THOSE logits (torch.topk on the two sides' own logits could differ wherever two
logits are one rounding apart). The logits are compared with an fp64 product (one rounding of an fp32-accumulated
sum: half an ulp of the dtype), the weights with an fp64 softmax of the kept logits (half an ulp).
"""

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from fma import KernelBackend, MoE, swiglu_packed
from fma.modules.moe.cuda_implementation import (
    build_routing_index,
    fused_router,
    router_topk_backward_cuda,
    router_topk_cuda,
)
from oracle import moe_oracle as O

from gpu_util import DEV, rel_err, to_np

pytestmark = pytest.mark.gpu

EPS = {torch.float16: 2.0**-10, torch.bfloat16: 2.0**-7}  # spacing of the dtype relative to the value, at most

SHAPES = [
    (7, 2048, 8, 2),
    (16384, 4096, 8, 2),  # the Mixtral-like benchmark layer
    (4099, 2048, 64, 8),  # fine-grained shape, a ragged last workgroup
    (32768, 2048, 64, 8),  # the fine-grained benchmark layer at full size
    (2050, 4096, 128, 8),  # large-E shape with few tokens: 32-token workgroups
    (8192, 4096, 128, 8),  # the large-E benchmark layer at full size
    (16400, 1024, 128, 8),  # enough tokens for 64-token workgroups, ragged end
    (300, 640, 200, 5),  # 128 < E <= 256: two passes over the activations
    (33, 200, 6, 4),  # H not a multiple of the 128-element step
    (100, 8, 3, 1),  # H smaller than one step, top-1
    (64, 512, 24, 3),
    (50, 576, 100, 7),
    (40, 1032, 300, 16),
    (20, 264, 1024, 64),  # both limits
    (5, 136, 1, 1),
    (19, 64, 16, 16),  # top_k == E
]


def _run_forward(x, w, k, with_counts=True, block_hist=None):
    T, E = x.size(0), w.size(0)
    logits = torch.full((T, E), float("nan"), device=DEV, dtype=x.dtype)
    weights = torch.full((T, k), float("nan"), device=DEV, dtype=x.dtype)
    selected = torch.full((T, k), -1, device=DEV, dtype=torch.int32)
    counts = torch.full((E,), 12345, device=DEV, dtype=torch.int32).view(torch.uint32) if with_counts else None
    router_topk_cuda(x, w, k, logits, weights, selected, counts, block_hist)
    torch.cuda.synchronize()
    return logits, weights, selected, counts


def _block_hist_buffer(T, E):
    return torch.full(((T + 15) // 16, E), 12345, device=DEV, dtype=torch.int32).view(torch.uint32)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,H,E,k", SHAPES)
def test_router_forward(dtype, T, H, E, k):
    torch.manual_seed(T + E)
    x = torch.randn(T, H).to(dtype)
    w = (torch.randn(E, H) / H**0.5).to(dtype)
    logits, weights, selected, counts = _run_forward(x.to(DEV), w.to(DEV), k)
    logits, weights, selected = logits.cpu(), weights.cpu(), selected.cpu()

    # logits: F.linear without bias (fma/modules/moe/__init__.py:193), one rounding
    ref = x.double() @ w.double().T
    err = (logits.double() - ref).abs()
    assert bool((err <= 0.5 * EPS[dtype] * ref.abs() + 1e-5).all()), f"logits off by {float(err.max())}"

    # expert choice: exact, from the returned logits
    expect_sel = O.topk_lowest_index_first(logits.float().numpy(), k)
    assert np.array_equal(selected.numpy(), expect_sel)

    # weights: softmax over the kept logits in fp32, then the cast (:199-200)
    kept = logits.double().gather(1, selected.long())
    ref_w = torch.softmax(kept, dim=-1)
    err = (weights.double() - ref_w).abs()
    assert bool((err <= 0.5005 * EPS[dtype] * ref_w + 1e-7).all()), f"weights off by {float(err.max())}"
    assert torch.equal(O.router_from_logits(logits, k)[1], selected.long())

    # histogram of the choice: what continuous_count returns for it (:215-217)
    assert np.array_equal(to_np(counts), O.continuous_count(selected.numpy().reshape(-1), E))

    # and without the optional histogram the other outputs are the same bits
    l2, w2, s2, _ = _run_forward(x.to(DEV), w.to(DEV), k, with_counts=False)
    assert torch.equal(l2.cpu(), logits) and torch.equal(w2.cpu(), weights) and torch.equal(s2.cpu(), selected)

    # the histogram per block of 16 tokens (with and without the total beside it), and the index built from it:
    # the same five arrays as from the ids alone
    for with_counts in (False, True):
        hist = _block_hist_buffer(T, E)
        l3, w3, s3, c3 = _run_forward(x.to(DEV), w.to(DEV), k, with_counts=with_counts, block_hist=hist)
        assert torch.equal(l3.cpu(), logits) and torch.equal(w3.cpu(), weights) and torch.equal(s3.cpu(), selected)
        expect_hist = np.zeros(((T + 15) // 16, E), dtype=np.int64)
        np.add.at(expect_hist, (np.repeat(np.arange(T) // 16, k), selected.numpy().reshape(-1)), 1)
        assert np.array_equal(to_np(hist).astype(np.int64), expect_hist)
        if with_counts:
            assert np.array_equal(to_np(c3), to_np(counts))
    plain = build_routing_index(s3, E)
    from_hist = build_routing_index(s3, E, token_block_histogram=hist)
    for a, b, name in zip(from_hist, plain, ("counts", "offsets", "perm", "eid", "inv")):
        assert torch.equal(a.view(torch.int32), b.view(torch.int32)), name


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_router_with_exact_logits_and_many_ties(dtype):
    # small-integer operands: fp32 accumulation is exact, logits are integers below 256 (exact in both dtypes) and
    # most rows hold several equal logits, so the order among equals is what is being checked
    rng = np.random.default_rng(3)
    T, H, E, k = 1000, 256, 40, 6
    x = torch.from_numpy(rng.integers(-2, 3, (T, H)).astype(np.float32))
    w = torch.from_numpy(rng.integers(-1, 2, (E, H)).astype(np.float32))
    logits, weights, selected, counts = _run_forward(x.to(dtype).to(DEV), w.to(dtype).to(DEV), k)
    exact = (x.long() @ w.long().T).float()
    assert float(exact.abs().max()) < 256
    assert torch.equal(logits.cpu().float(), exact)
    expect_sel = O.topk_lowest_index_first(exact.numpy(), k)
    ties = sum(len(set(row[s] for s in sel)) < k for row, sel in zip(exact.numpy(), expect_sel))
    assert ties > T // 4, "the case is meant to be tie-heavy"
    assert np.array_equal(selected.cpu().numpy(), expect_sel)
    # the values selected are the ones torch.topk selects on the GPU
    assert torch.equal(
        logits.gather(1, selected.long()).cpu(), torch.topk(logits.float(), k, dim=-1).values.to(dtype).cpu()
    )


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize(
    "T,E,k", [(7, 8, 2), (1000, 8, 2), (513, 64, 8), (300, 128, 8), (100, 3, 1), (77, 300, 16), (20, 1024, 64), (31, 65, 36)]
)
@pytest.mark.parametrize("which", ["both", "weights", "logits"])
def test_router_backward(dtype, T, E, k, which):
    torch.manual_seed(E + k)
    logits = torch.randn(T, E).to(dtype)
    _, selected = O.router_from_logits(logits, k)
    dw = torch.randn(T, k).to(dtype) if which != "logits" else None
    dl = torch.randn(T, E).to(dtype) if which != "weights" else None

    out = torch.full((T, E), float("nan"), device=DEV, dtype=dtype)
    router_topk_backward_cuda(
        logits.to(DEV), selected.int().to(DEV), None if dw is None else dw.to(DEV), None if dl is None else dl.to(DEV), out
    )
    got = out.cpu().double()

    # unrounded answer in fp64: direct term + s * (dw - <s, dw>) at the kept columns
    ref = torch.zeros(T, E, dtype=torch.float64) if dl is None else dl.double().clone()
    if dw is not None:
        s = torch.softmax(logits.double().gather(1, selected), dim=-1)
        ds = s * (dw.double() - (s * dw.double()).sum(-1, keepdim=True))
        # two roundings on the kept columns (the softmax gradient, then the sum), one elsewhere (none: a copy)
        ref_lo = ref.clone().scatter_add(1, selected, ds)
        tol = torch.zeros(T, E, dtype=torch.float64).scatter_add(
            1, selected, 0.5 * EPS[dtype] * ds.abs() + 1e-7
        ) + (0.5 * EPS[dtype] * ref_lo.abs() if dl is not None else 0.0)
        ref = ref_lo
    else:
        tol = torch.zeros(T, E, dtype=torch.float64)
    assert bool(((got - ref).abs() <= tol * 1.001).all()), f"max excess {float(((got - ref).abs() - tol).max())}"
    # columns that were not chosen carry the direct term unchanged (or zero)
    untouched = torch.ones(T, E, dtype=torch.bool).scatter(1, selected, False)
    direct = torch.zeros(T, E, dtype=torch.float64) if dl is None else dl.double()
    assert torch.equal(got[untouched], direct[untouched])

    # and the oracle's autograd in the same dtype. Same rounding points, but the two fp32 evaluations of
    # s * (dw - <s, dw>) differ in the last places, which can move the 16-bit rounding of that intermediate by one of ITS
    # units (larger than a unit of the final sum where the direct term cancels it) and the rounding of the sum by one more.
    auto = O.router_logits_grad(logits, selected, dw, dl).double()
    slack = torch.full((T, E), 2e-6, dtype=torch.float64)
    if dw is not None:
        slack = slack.scatter_add(1, selected, EPS[dtype] * ds.abs() + 2e-6 * float(dw.abs().max()))
    assert bool(((got - auto).abs() <= EPS[dtype] * auto.abs() + slack).all())


def test_router_autograd_matches_unfused_router():
    # the whole router through autograd: fused function against the reference's formulation in ATen on the same
    # device, with the discrete choice shared, for x, the gate weight and both outputs
    torch.manual_seed(11)
    T, H, E, k = 512, 1024, 16, 4
    x = torch.randn(T, H).bfloat16().to(DEV)
    w = (torch.randn(E, H) / H**0.5).bfloat16().to(DEV)
    dl = torch.randn(T, E).bfloat16().to(DEV)
    dw = torch.randn(T, k).bfloat16().to(DEV)

    xa, wa = x.clone().requires_grad_(), w.clone().requires_grad_()
    logits, weights, selected = fused_router(xa, wa, k)
    assert not selected.requires_grad and selected.dtype == torch.int32
    torch.autograd.backward([logits, weights], [dl, dw])

    xb, wb = x.float().requires_grad_(), w.float().requires_grad_()
    ref_logits = F.linear(xb, wb)
    ref_weights = torch.softmax(ref_logits.gather(1, selected.long()), dim=-1)
    torch.autograd.backward([ref_logits, ref_weights], [dl.float(), dw.float()])

    for name, a, b in [("x grad", xa.grad, xb.grad), ("gate weight grad", wa.grad, wb.grad)]:
        max_rel, frob_rel = rel_err(a, b)
        assert max_rel <= 2e-2 and frob_rel <= 1e-2, f"{name}: max_rel={max_rel:.4g} frob_rel={frob_rel:.4g}"

    # only one of the two outputs used
    for use in (0, 1):
        xa.grad = wa.grad = None
        outs = fused_router(xa, wa, k)
        outs[use].backward([dl, dw][use])
        assert xa.grad is not None and bool(torch.isfinite(xa.grad).all())


def test_moe_layer_with_and_without_fused_router():
    torch.manual_seed(5)
    E, k, H, I, T = 8, 2, 512, 1024, 256
    moe = MoE(E, k, H, I, swiglu_packed, True, False, 0.02).to(torch.bfloat16).to(DEV)
    x = torch.randn(T, H).bfloat16().to(DEV)
    dy = torch.randn(T, H).bfloat16().to(DEV)
    results = []
    for fuse in (True, False):
        moe.fuse_router = fuse
        moe.zero_grad()
        xi = x.clone().requires_grad_()
        y, logits = moe(xi, kernel_backend=KernelBackend.cuda)
        (y * dy).sum().backward()
        results.append((y, logits, xi.grad, moe.gate.weight.grad.clone(), moe._compute_routing_weights(x)[2]))
    fused, plain = results
    # the two gate GEMMs may round a logit differently; compare tokens whose choice agrees (nearly all)
    same = (fused[4].long() == plain[4].long()).all(-1)
    assert float(same.float().mean()) > 0.97
    max_rel, _ = rel_err(fused[1], plain[1])
    assert max_rel <= 2.0**-7
    for a, b in [(fused[0][same], plain[0][same]), (fused[2][same], plain[2][same])]:
        max_rel, frob_rel = rel_err(a, b)
        assert max_rel <= 3e-2 and frob_rel <= 1e-2
    if bool(same.all()):
        max_rel, frob_rel = rel_err(fused[3], plain[3])
        assert max_rel <= 3e-2 and frob_rel <= 1.5e-2


def test_router_rejects_bad_arguments():
    x = torch.zeros(4, 64, device=DEV, dtype=torch.bfloat16)
    w = torch.zeros(8, 64, device=DEV, dtype=torch.bfloat16)

    def call(x, w, k):
        T, E = x.size(0), w.size(0)
        router_topk_cuda(
            x, w, k, torch.empty(T, E, device=DEV, dtype=x.dtype), torch.empty(T, k, device=DEV, dtype=x.dtype),
            torch.empty(T, k, device=DEV, dtype=torch.int32), None, None,
        )

    with pytest.raises(RuntimeError, match="top_k"):
        call(x, w, 9)
    with pytest.raises(RuntimeError, match="multiple of 8"):
        call(x[:, :60].contiguous(), w[:, :60].contiguous(), 2)
    with pytest.raises(RuntimeError, match="dtype"):
        call(x.float(), w.float(), 2)
    call(x[:0], w, 2)  # no tokens: nothing to do
