"""GPU parity of the fp32 path: the grouped GEMM on fp32 operands and the MoE layer in fp32 (the reference runs its
kernel backends in fp32 too, tests/modules/moe_test.py:100-150: output atol 6e-3, input gradient 6.5e-3, weight
gradients 3e-2 — its Triton matrix products use TF32; here the products are true fp32, so the same cases are held to
bars a hundred times tighter), including the small CPU-runnable configuration against the golden fixture."""

import os

import numpy as np
import pytest
import torch
import torch.nn as nn

from fma import KernelBackend, MoE, grouped_gemm, swiglu_packed
from oracle import moe_oracle as O

from gpu_util import DEV, rel_err

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _u32(values):
    return torch.tensor(values, dtype=torch.int64).to(torch.uint32).to(DEV)


def _operands(M_list, N_list, K_list, tA, tB, seed, integer):
    g = torch.Generator().manual_seed(seed)
    As, Bs = [], []
    for M, N, K in zip(M_list, N_list, K_list):
        sa, sb = ((K, M) if tA else (M, K)), ((N, K) if tB else (K, N))
        if integer:
            As.append(torch.randint(-8, 9, sa, generator=g).float())
            Bs.append(torch.randint(-8, 9, sb, generator=g).float())
        else:
            As.append(torch.randn(sa, generator=g))
            Bs.append(torch.randn(sb, generator=g))
    return torch.cat([a.reshape(-1) for a in As]), torch.cat([b.reshape(-1) for b in Bs])


def _run(A, B, M_list, N_list, K_list, tA, tB, alpha=1.0):
    return grouped_gemm(
        A=A.to(DEV), B=B.to(DEV), C=None, M_array=_u32(M_list), N_array=_u32(N_list), K_array=_u32(K_list),
        output_shape=(sum(m * n for m, n in zip(M_list, N_list)),), alpha=alpha, is_A_transposed=tA, is_B_transposed=tB,
    )


SHAPES = [
    ([8], [8], [8]),
    ([128], [128], [16]),
    ([1, 7, 13], [24, 24, 24], [40, 40, 40]),
    ([264, 0, 8, 520, 1000], [264] * 5, [200] * 5),  # an empty group, tails in every dimension
    ([3, 129, 65], [1, 130, 257], [5, 17, 33]),  # nothing aligned to anything, N and K differ per group
    ([300, 300], [512, 512], [72, 0]),  # a group without a reduction dimension: zeros
    ([64] * 40, [96] * 40, [48] * 40),
]


@pytest.mark.parametrize("tA", [False, True])
@pytest.mark.parametrize("tB", [False, True])
@pytest.mark.parametrize("M_list,N_list,K_list", SHAPES)
def test_fp32_integer_known_answer(tA, tB, M_list, N_list, K_list):
    # the reference's construction (tests/ops/grouped_gemm_test.py:38-92) in fp32: integer operands in [-8, 8], every
    # partial sum is an integer below 2^24, so any summation order gives the exact product
    A, B = _operands(M_list, N_list, K_list, tA, tB, seed=11, integer=True)
    expect = O.grouped_gemm(A, B, M_list, N_list, K_list, tA, tB)
    got = _run(A, B, M_list, N_list, K_list, tA, tB)
    assert got.dtype == torch.float32 and got.shape == expect.shape
    assert torch.equal(got.cpu(), expect)


@pytest.mark.parametrize("tA,tB", [(False, True), (False, False), (True, False), (True, True)])
def test_fp32_random_operands_and_alpha(tA, tB):
    M_list, N_list, K_list = [500, 37, 0, 1024], [384, 200, 64, 520], [1000, 333, 8, 2048]
    A, B = _operands(M_list, N_list, K_list, tA, tB, seed=12, integer=False)
    got = _run(A, B, M_list, N_list, K_list, tA, tB, alpha=0.37).cpu().double()
    # the product in fp64 (the oracle function itself accumulates in fp32, like the kernel)
    outs, oa, ob = [], 0, 0
    for M, N, K in zip(M_list, N_list, K_list):
        a = A[oa : oa + M * K].double().reshape((K, M) if tA else (M, K))
        b = B[ob : ob + K * N].double().reshape((N, K) if tB else (K, N))
        outs.append((0.37 * ((a.T if tA else a) @ (b.T if tB else b))).reshape(-1))
        oa, ob = oa + M * K, ob + K * N
    expect = torch.cat(outs)
    # fp32 accumulation, in reduction order, of up to 2048 products of N(0,1) numbers: the rounding errors of the
    # partial sums (magnitude up to ~200, spacing 1.5e-5) add up like a random walk
    assert float((got - expect).abs().max()) <= 5e-6 * float(expect.abs().max())
    assert float((got - expect).norm()) <= 1e-6 * float(expect.norm())
    # and the oracle (fp32 accumulation in another order) agrees to the same bar
    oracle = O.grouped_gemm(A, B, M_list, N_list, K_list, tA, tB, alpha=0.37).double()
    assert float((got - oracle).abs().max()) <= 5e-6 * float(expect.abs().max())


def test_fp32_reference_shape_and_many_tiles_per_workgroup():
    # the reference's test shape (E=16, sum(M)=65536, N=512, K=4096) scaled to keep the host-side product short
    torch.manual_seed(42)
    E, N, K = 16, 512, 1024
    cuts = sorted(torch.randint(0, 16384, (E - 1,)).tolist())
    M_list = [b - a for a, b in zip([0] + cuts, cuts + [16384])]
    A, B = _operands(M_list, [N] * E, [K] * E, False, True, seed=13, integer=True)
    got = _run(A, B, M_list, [N] * E, [K] * E, False, True)
    expect = torch.cat(
        [(a.to(DEV) @ b.to(DEV).T).reshape(-1) for a, b in zip(A.reshape(-1, K).split(M_list), B.reshape(E, N, K))]
    )
    assert torch.equal(got, expect)


def _glu(x):
    a, b = x.chunk(2, dim=-1)
    return a * torch.sigmoid(b)


@pytest.mark.parametrize("E,k,H,I", [(2, 2, 2048, 8192), (8, 2, 2048, 8192), (8, 4, 2048, 8192), (128, 8, 576, 256)])
@pytest.mark.parametrize("act_name", ["swiglu", "glu", "gelu"])
def test_moe_reference_cases_fp32(E, k, H, I, act_name):
    torch.manual_seed(42)
    is_glu = act_name != "gelu"
    act = {"swiglu": swiglu_packed, "glu": nn.GLU(), "gelu": nn.GELU(approximate="tanh")}[act_name]
    oracle_act = {"swiglu": O.swiglu_packed, "glu": _glu, "gelu": nn.GELU(approximate="tanh")}[act_name]
    moe = MoE(E, k, H, I, act, is_glu, False, 0.02).to(DEV)
    x = torch.randn(7, H, device=DEV).requires_grad_()
    y, logits = moe(x, kernel_backend=KernelBackend.cuda)
    assert y.dtype == torch.float32
    y.sum().backward()

    with torch.no_grad():
        _, _, selected = moe._compute_routing_weights(x.detach())
    selected = selected.cpu().long()
    xf = x.detach().cpu().requires_grad_()
    w1 = moe.c_fc.weight.detach().cpu().requires_grad_()
    w2 = moe.c_proj.weight.detach().cpu().requires_grad_()
    values = torch.nn.functional.linear(xf, moe.gate.weight.detach().cpu()).gather(1, selected)
    weights = torch.softmax(values, dim=-1)
    yo = O.moe_experts(xf, weights, selected, w1, w2, oracle_act)
    yo.sum().backward()
    for name, a, b, atol in [
        ("output", y, yo, 6e-5), ("input gradient", x.grad, xf.grad, 6.5e-5),
        ("c_fc weight gradient", moe.c_fc.weight.grad, w1.grad, 3e-4), ("c_proj weight gradient", moe.c_proj.weight.grad, w2.grad, 3e-4),
    ]:
        err = float((a.detach().cpu() - b.detach()).abs().max())
        assert err <= atol, f"{name}: {err}"


def test_small_configuration_in_fp32_against_golden_fixture():
    # T=512, H=256, I=512, E=8, k=2 entirely in fp32, as the fixture was computed (tests/golden/make_golden.py)
    from golden.make_golden import c1_inputs

    fx = np.load(os.path.join(GOLDEN, "c1_moe_fp32.npz"))
    x, wg, w1, w2 = c1_inputs()
    moe = MoE(8, 2, 256, 512, swiglu_packed, True, False, 0.02)
    with torch.no_grad():
        moe.gate.weight.copy_(wg)
        moe.c_fc.weight.copy_(w1)
        moe.c_proj.weight.copy_(w2)
    moe = moe.to(DEV)
    xd = x.to(DEV).requires_grad_()
    # the fixture differentiates the expert path for fixed routing weights (computed from a detached input)
    with torch.no_grad():
        _, weights, selected = moe._compute_routing_weights(xd.detach())
    assert np.array_equal(selected.cpu().numpy(), fx["selected"]), "routing differs from the fixture"
    assert float((weights.cpu() - torch.from_numpy(fx["router_weights"])).abs().max()) <= 1e-6
    y = moe._compute_experts(xd, weights, selected, KernelBackend.cuda)
    y.sum().backward()
    for got, key in [(y, "y"), (xd.grad, "dx"), (moe.c_fc.weight.grad[:, ::16, ::8], "dw1_sample"), (moe.c_proj.weight.grad[:, ::8, ::16], "dw2_sample")]:
        max_rel, frob_rel = rel_err(got, torch.from_numpy(fx[key]))
        assert max_rel <= 2e-5 and frob_rel <= 5e-6, f"{key}: max_rel={max_rel:.3g} frob_rel={frob_rel:.3g}"
