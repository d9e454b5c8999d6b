"""GPU parity of the per-expert bias (fma_expert_bias_add / fma_expert_bias_grad) and of the MoE layer with
add_bias=True against the oracle's per-expert F.linear(x_e, W[e], bias[e]) (fma/modules/moe/__init__.py:98-105)."""

import pytest
import torch
import torch.nn as nn

from fma import KernelBackend, MoE, swiglu_packed
from fma.modules.moe.cuda_implementation import expert_bias_add_cuda, expert_bias_grad_cuda
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
    assert not moe.fuse_swiglu  # the fused epilogue has no bias term
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
