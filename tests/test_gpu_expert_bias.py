"""GPU parity of the per-expert bias (fma_expert_bias_add / fma_expert_bias_grad) and of the MoE layer with
add_bias=True against the oracle's per-expert F.linear(x_e, W[e], bias[e]) (fma/modules/moe/__init__.py:98-105)."""

import pytest
import torch
import torch.nn as nn

from fma import KernelBackend, MoE, swiglu_packed
from fma.modules.moe.cuda_implementation import (
    expert_bias_add_cuda,
    expert_bias_grad_cuda,
    grouped_gemm_ragged_cuda,
    grouped_gemm_swiglu_cuda,
)
from oracle import moe_oracle as O

from gpu_util import DEV, rel_err

pytestmark = pytest.mark.gpu

CASES = [
    # counts per expert, N
    ([5, 0, 3, 1], 64),
    ([0, 0, 7], 8),
    ([300, 1, 0, 4095, 17, 0, 256, 2], 4096),
    ([100] * 128, 1536),
    ([4096, 1, 3000, 0, 3], 28672),
    ([1], 16),
]


def _counts_tensor(counts):
    return torch.tensor(counts, dtype=torch.int32).view(torch.uint32).to(DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("counts,N", CASES)
def test_bias_add_is_the_rounded_fp32_sum(dtype, counts, N):
    torch.manual_seed(N + len(counts))
    R, E = sum(counts), len(counts)
    y = torch.randn(R + 3, N).to(dtype)  # three rows past the last group must stay untouched
    bias = torch.randn(E, N).to(dtype)
    expect = y.clone()
    expect[:R] = (y[:R].float() + bias.float().repeat_interleave(torch.tensor(counts), dim=0)).to(dtype)
    y_d = y.to(DEV)
    expert_bias_add_cuda(y_d, bias.to(DEV), _counts_tensor(counts))
    assert torch.equal(y_d.cpu(), expect)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("counts,N", CASES)
def test_bias_grad_is_the_segmented_column_sum(dtype, counts, N):
    torch.manual_seed(N + len(counts))
    R, E = sum(counts), len(counts)
    dy = torch.randn(R, N).to(dtype)
    got = torch.full((E, N), float("nan"), dtype=dtype, device=DEV)
    expert_bias_grad_cuda(dy.to(DEV), _counts_tensor(counts), got)
    again = torch.full((E, N), float("nan"), dtype=dtype, device=DEV)
    expert_bias_grad_cuda(dy.to(DEV), _counts_tensor(counts), again)
    assert torch.equal(got, again), "the summation order is fixed: same bits on every call"

    expect = torch.stack([seg.double().sum(0) for seg in dy.split(counts, dim=0)])
    eps = {torch.float32: 2.0**-23, torch.float16: 2.0**-10, torch.bfloat16: 2.0**-7}[dtype]
    # one rounding to the dtype of an fp32-accumulated sum of up to a few hundred rows per slice
    mags = torch.stack([seg.double().abs().sum(0) for seg in dy.split(counts, dim=0)])
    tol = 0.5 * eps * expect.abs() * 1.001 + 2.0**-21 * mags + 1e-30
    assert bool(((got.cpu().double() - expect).abs() <= tol).all())
    for e, c in enumerate(counts):
        if c == 0:
            assert float(got[e].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize(
    "counts,N,K",
    [
        ([300, 1, 0, 4095, 17, 0, 256, 2], 4096, 512),  # thin groups, empty groups, 16 column tiles
        ([2048 + 8 * (e % 7) for e in range(24)], 1024, 512),  # every workgroup streams through several tiles
        ([40] * 64, 136, 192),  # half-width tiles, a last column tile of 8 columns, 3 K steps
        ([1000, 520, 8], 264, 64),  # one K step per tile; columns end inside a tile
        ([700, 0, 33], 512, 0),  # no reduction at all: the output is the bias
    ],
)
def test_bias_in_the_gemm_epilogue_equals_gemm_then_bias_add(dtype, counts, N, K):
    torch.manual_seed(N + K)
    R, E = sum(counts), len(counts)
    x = torch.randn(R, K, device=DEV).to(dtype)
    w = (torch.randn(E, N, K, device=DEV) * 0.2).to(dtype)
    bias = torch.randn(E, N, device=DEV).to(dtype)
    M = _counts_tensor(counts)
    two_pass = torch.full((R, N), 7.0, dtype=dtype, device=DEV)
    grouped_gemm_ragged_cuda(x, w, two_pass, M, False, 0, N, K, False, True)
    expert_bias_add_cuda(two_pass, bias, M)
    fused = torch.full((R, N), 7.0, dtype=dtype, device=DEV)
    grouped_gemm_ragged_cuda(x, w, fused, M, False, 0, N, K, False, True, bias)
    assert torch.equal(fused, two_pass)
    # and against the definition: per-expert linear in fp64, rounded, plus the bias, rounded
    off = 0
    for e, c in enumerate(counts):
        if c and c <= 1000:
            y = (x[off:off + c].double() @ w[e].double().T).to(dtype)
            expect = (y.float() + bias[e].float()).to(dtype)
            # (the fp32-accumulated product may round to the neighbour of the fp64 one: one step of the product's size)
            eps = 2.0 ** (-7 if dtype == torch.bfloat16 else -10)
            bad = (fused[off:off + c].float() - expect.float()).abs() > eps * (y.float().abs() + expect.float().abs()) + 1e-3
            assert int(bad.sum()) == 0
        off += c


@pytest.mark.parametrize("counts,I,K", [([100, 0, 300, 1], 128, 64), ([40] * 16, 72, 520), ([3000, 0, 5000, 1, 4999], 1408, 520)])
def test_bias_in_the_fused_swiglu_epilogue(counts, I, K):
    torch.manual_seed(I + K)
    R, E = sum(counts), len(counts)
    x = torch.randn(R, K, device=DEV).bfloat16()
    w = (torch.randn(E, 2 * I, K, device=DEV) * 0.1).bfloat16()
    bias = torch.randn(E, 2 * I, device=DEV).bfloat16()
    M = _counts_tensor(counts)
    h_ref = torch.empty(R, 2 * I, dtype=torch.bfloat16, device=DEV)
    grouped_gemm_ragged_cuda(x, w, h_ref, M, False, 0, 2 * I, K, False, True)
    expert_bias_add_cuda(h_ref, bias, M)
    h = torch.empty_like(h_ref)
    act = torch.empty(R, I, dtype=torch.bfloat16, device=DEV)
    grouped_gemm_swiglu_cuda(x, w, M, h, act, bias)
    assert torch.equal(h, h_ref)
    assert torch.equal(act, swiglu_packed(h_ref))
    act_only = torch.empty_like(act)
    grouped_gemm_swiglu_cuda(x, w, M, None, act_only, bias)
    assert torch.equal(act_only, act)


def test_bias_in_the_epilogue_is_refused_outside_the_forward_form():
    x = torch.zeros(64, 64, device=DEV, dtype=torch.bfloat16)
    out = torch.zeros(64, 64, device=DEV, dtype=torch.bfloat16)
    bias = torch.zeros(1, 64, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="forward form"):
        grouped_gemm_ragged_cuda(x, x, out, _counts_tensor([64]), False, 0, 64, 64, False, False, bias)
    with pytest.raises(RuntimeError, match="forward form"):
        grouped_gemm_ragged_cuda(x, x, out, _counts_tensor([64]), True, 64, 64, 0, False, True, bias)


def _glu(x):
    a, b = x.chunk(2, dim=-1)
    return a * torch.sigmoid(b)


@pytest.mark.parametrize("act_name", ["swiglu", "glu", "gelu"])
@pytest.mark.parametrize("E,k,H,I,T", [(4, 2, 256, 512, 7), (8, 2, 512, 1024, 300), (128, 8, 576, 256, 64)])
def test_moe_layer_with_bias(act_name, E, k, H, I, T):
    torch.manual_seed(42)
    is_glu = act_name != "gelu"
    act = {"swiglu": swiglu_packed, "glu": nn.GLU(), "gelu": nn.GELU(approximate="tanh")}[act_name]
    oracle_act = {"swiglu": O.swiglu_packed, "glu": _glu, "gelu": nn.GELU(approximate="tanh")}[act_name]
    moe = MoE(E, k, H, I, act, is_glu, True, 0.02).to(torch.bfloat16).to(DEV)
    assert moe.fuse_swiglu == (act_name == "swiglu")  # the fused epilogue adds the bias before the activation
    with torch.no_grad():  # reset_parameters zeroes the biases (fma/modules/moe/__init__.py:121-122)
        moe.c_fc.bias.normal_(0, 0.5)
        moe.c_proj.bias.normal_(0, 0.5)
    x = torch.randn(T, H).bfloat16().to(DEV).requires_grad_()
    dy = torch.randn(T, H).bfloat16().to(DEV)
    y, _ = moe(x, kernel_backend=KernelBackend.cuda)
    y.backward(dy)

    # the oracle in fp32 on the same parameters, with the module's discrete choice
    with torch.no_grad():
        _, _, selected = moe._compute_routing_weights(x.detach())
    selected = selected.cpu().long()
    xf = x.detach().cpu().float().requires_grad_()
    params = [p.detach().cpu().float().requires_grad_() for p in (moe.c_fc.weight, moe.c_proj.weight, moe.c_fc.bias, moe.c_proj.bias)]
    values = torch.nn.functional.linear(xf, moe.gate.weight.detach().cpu().float()).gather(1, selected)
    weights = torch.softmax(values, dim=-1)
    yo = O.moe_experts(xf, weights, selected, params[0], params[1], oracle_act, params[2], params[3])
    yo.backward(dy.cpu().float())

    got = [y, x.grad, moe.c_fc.weight.grad, moe.c_proj.weight.grad, moe.c_fc.bias.grad, moe.c_proj.bias.grad]
    ref = [yo, xf.grad] + [p.grad for p in params]
    names = ["output", "input gradient", "c_fc weight gradient", "c_proj weight gradient", "c_fc bias gradient", "c_proj bias gradient"]
    for name, a, b in zip(names, got, ref):
        max_rel, frob_rel = rel_err(a.detach(), b.detach())
        assert max_rel <= 3e-2 and frob_rel <= 1.5e-2, f"{name}: max_rel={max_rel:.4g} frob_rel={frob_rel:.4g}"
    # the bias really took part: without it the output differs
    with torch.no_grad():
        moe.c_proj.bias.zero_()
        y0, _ = moe(x.detach(), kernel_backend=KernelBackend.cuda)
    assert float((y0 - y.detach()).abs().max()) > 0.05


def test_bias_ops_reject_bad_arguments():
    y = torch.zeros(4, 12, device=DEV, dtype=torch.bfloat16)  # 24-byte rows
    with pytest.raises(RuntimeError, match="multiple of 16"):
        expert_bias_add_cuda(y, torch.zeros(2, 12, device=DEV, dtype=torch.bfloat16), _counts_tensor([2, 2]))
    with pytest.raises(RuntimeError):
        expert_bias_add_cuda(y.cpu(), torch.zeros(2, 12, dtype=torch.bfloat16), torch.zeros(2, dtype=torch.int32).view(torch.uint32))
