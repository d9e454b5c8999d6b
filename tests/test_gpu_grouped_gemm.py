"""GPU parity of the grouped GEMM: exact on integer-valued operands (every layout, ragged / empty / one-row groups),
within bf16 rounding on random operands, and the fused SwiGLU epilogue bit-identical to GEMM followed by swiglu."""

import pytest
import torch

from fma import grouped_gemm, swiglu_packed
from fma.modules.moe.cuda_implementation import grouped_gemm_swiglu_cuda
from oracle import moe_oracle as O

from gpu_util import DEV, rel_err

pytestmark = pytest.mark.gpu


def _u32(values):
    return torch.tensor(values, dtype=torch.int64).to(torch.uint32).to(DEV)


def _integer_operands(M_list, N_list, K_list, tA, tB, seed):
    g = torch.Generator().manual_seed(seed)
    As, Bs = [], []
    for M, N, K in zip(M_list, N_list, K_list):
        As.append(torch.randint(-8, 9, (K, M) if tA else (M, K), generator=g).to(torch.bfloat16))
        Bs.append(torch.randint(-8, 9, (N, K) if tB else (K, N), generator=g).to(torch.bfloat16))
    return torch.cat([a.reshape(-1) for a in As]), torch.cat([b.reshape(-1) for b in Bs])


@pytest.mark.parametrize("tA", [False, True])
@pytest.mark.parametrize("tB", [False, True])
@pytest.mark.parametrize(
    "M_list,N,K",
    [
        ([8], 8, 8),
        ([256], 256, 64),
        ([264, 0, 8, 520, 1000], 264, 200),  # empty group, tails in every dimension
        ([1, 7, 13], 24, 40),  # M not a multiple of 8 (for tA that is the contiguous dimension: scalar path)
        ([300, 300], 512, 72),
        ([16, 16], 20, 36),  # N, K not multiples of 8: scalar path
    ],
)
def test_integer_known_answer_small(tA, tB, M_list, N, K):
    E = len(M_list)
    A, B = _integer_operands(M_list, [N] * E, [K] * E, tA, tB, seed=7)
    expect = O.grouped_gemm(A, B, M_list, [N] * E, [K] * E, tA, tB)
    got = grouped_gemm(
        A=A.to(DEV), B=B.to(DEV), C=None, M_array=_u32(M_list), N_array=_u32([N] * E), K_array=_u32([K] * E),
        output_shape=(sum(M_list) * N,), is_A_transposed=tA, is_B_transposed=tB,
    )
    assert got.shape == expect.shape and got.dtype == torch.bfloat16
    assert float((got.cpu().float() - expect.float()).abs().max()) == 0


@pytest.mark.parametrize("tA", [False, True])
@pytest.mark.parametrize("tB", [False, True])
def test_integer_known_answer_reference_shape(tA, tB):
    # the reference's test: E=16, sum(M)=65536, N=512, K=4096, operands integers in [-8, 8], max |diff| == 0
    # (tests/ops/grouped_gemm_test.py:38-92). Expected values: fp32 matmul on the GPU, exact for these operands
    # (|sum| <= 64*4096 < 2^24) in any summation order.
    torch.manual_seed(42)
    E, K, N = 16, 4096, 512
    M_list = [512, 3176, 2048] * 5 + [36856]
    As, Bs, Ds = [], [], []
    for M in M_list:
        a = torch.randint(-8, 9, (K, M) if tA else (M, K), device=DEV, dtype=torch.bfloat16)
        b = torch.randint(-8, 9, (N, K) if tB else (K, N), device=DEV, dtype=torch.bfloat16)
        As.append(a)
        Bs.append(b)
        Ds.append(((a.T if tA else a).float() @ (b.T if tB else b).float()).to(torch.bfloat16).reshape(-1))
    A = torch.cat([a.reshape(-1) for a in As])
    B = torch.cat([b.reshape(-1) for b in Bs])
    out = grouped_gemm(
        A=A, B=B, C=None, M_array=_u32(M_list), N_array=_u32([N] * E), K_array=_u32([K] * E),
        output_shape=(sum(M_list) * N,), is_A_transposed=tA, is_B_transposed=tB,
    )
    assert float((out.float() - torch.cat(Ds).float()).abs().max()) == 0


def test_varying_n_and_k_per_group_and_alpha():
    M_list, N_list, K_list = [40, 264, 8], [16, 520, 256], [64, 8, 136]
    A, B = _integer_operands(M_list, N_list, K_list, False, True, seed=9)
    expect = O.grouped_gemm(A, B, M_list, N_list, K_list, False, True, alpha=0.5)
    got = grouped_gemm(
        A=A.to(DEV), B=B.to(DEV), C=None, M_array=_u32(M_list), N_array=_u32(N_list), K_array=_u32(K_list),
        output_shape=(sum(m * n for m, n in zip(M_list, N_list)),), alpha=0.5, is_A_transposed=False,
        is_B_transposed=True,
    )
    assert torch.equal(got.cpu(), expect)


@pytest.mark.parametrize("tA,tB", [(False, True), (False, False), (True, False)])
def test_random_operands_within_bf16_rounding(tA, tB):
    # bf16 N(0,1) operands against fp32 math on the same bf16 values; the only difference is summation order in
    # fp32 and the final rounding to bf16: relative error of one bf16 ulp (2^-8) of the largest output
    torch.manual_seed(5)
    M_list, N, K = [700, 3, 1029, 0, 256], 384, 1536
    E = len(M_list)
    As = [torch.randn((K, M) if tA else (M, K)).bfloat16() for M in M_list]
    Bs = [torch.randn((N, K) if tB else (K, N)).bfloat16() for _ in M_list]
    A = torch.cat([a.reshape(-1) for a in As])
    B = torch.cat([b.reshape(-1) for b in Bs])
    expect = O.grouped_gemm(A.float(), B.float(), M_list, [N] * E, [K] * E, tA, tB)
    got = grouped_gemm(
        A=A.to(DEV), B=B.to(DEV), C=None, M_array=_u32(M_list), N_array=_u32([N] * E), K_array=_u32([K] * E),
        output_shape=(sum(M_list) * N,), is_A_transposed=tA, is_B_transposed=tB,
    )
    max_rel, frob_rel = rel_err(got, expect)
    assert max_rel <= 2**-8 and frob_rel <= 2**-8


@pytest.mark.parametrize(
    "M_list,I,K",
    [([100, 0, 300, 1], 128, 64), ([512, 260], 1408, 256), ([40] * 16, 72, 520), ([3000, 0, 5000, 7000, 1, 4999], 1408, 520)],
)
def test_fused_swiglu_equals_gemm_then_swiglu(M_list, I, K):
    torch.manual_seed(I)
    E, R = len(M_list), sum(M_list)
    x = torch.randn(R, K).bfloat16().to(DEV)
    w = (torch.randn(E, 2 * I, K) * 0.1).bfloat16().to(DEV)
    M = _u32(M_list)
    h = torch.empty(R, 2 * I, dtype=torch.bfloat16, device=DEV)
    act = torch.empty(R, I, dtype=torch.bfloat16, device=DEV)
    grouped_gemm_swiglu_cuda(x, w, M, h, act)
    h_ref = grouped_gemm(
        A=x, B=w, C=None, M_array=M, N_array=_u32([2 * I] * E), K_array=_u32([K] * E), output_shape=(R, 2 * I),
        is_A_transposed=False, is_B_transposed=True,
    )
    assert torch.equal(h, h_ref)
    assert torch.equal(act, swiglu_packed(h_ref))
    # against the oracle: per-expert linear, then up * silu(gate) with up = first half
    xs = x.cpu().float().split(M_list)
    expect = torch.cat([O.swiglu_packed((xs[e] @ w[e].cpu().float().T).bfloat16()) for e in range(E)])
    assert rel_err(act, expect)[0] <= 2**-7
    act_only = torch.empty_like(act)
    grouped_gemm_swiglu_cuda(x, w, M, None, act_only)
    assert torch.equal(act_only, act)


@pytest.mark.parametrize("tA,tB", [(False, True), (False, False), (True, False), (True, True)])
def test_fp16_integer_known_answer(tA, tB):
    # fp16 operands: integers in [-3, 3], K = 200, so every sum (|sum| <= 1800 < 2048) is exact in fp16
    M_list, N, K = [264, 0, 8, 520, 1000], 264, 200
    E = len(M_list)
    g = torch.Generator().manual_seed(11)
    As = [torch.randint(-3, 4, (K, M) if tA else (M, K), generator=g).to(torch.float16) for M in M_list]
    Bs = [torch.randint(-3, 4, (N, K) if tB else (K, N), generator=g).to(torch.float16) for _ in M_list]
    A = torch.cat([a.reshape(-1) for a in As])
    B = torch.cat([b.reshape(-1) for b in Bs])
    expect = O.grouped_gemm(A, B, M_list, [N] * E, [K] * E, tA, tB)
    got = grouped_gemm(
        A=A.to(DEV), B=B.to(DEV), C=None, M_array=_u32(M_list), N_array=_u32([N] * E), K_array=_u32([K] * E),
        output_shape=(sum(M_list) * N,), is_A_transposed=tA, is_B_transposed=tB,
    )
    assert got.dtype == torch.float16
    assert float((got.cpu().float() - expect.float()).abs().max()) == 0


def test_fp16_random_operands_and_fused_swiglu():
    # fp16 N(0,1) x 0.1 operands: one fp16 ulp (2^-11) of the largest output against fp32 math; the fused SwiGLU
    # epilogue equals GEMM followed by swiglu_packed bit for bit, as for bf16
    torch.manual_seed(6)
    M_list, I, K = [300, 0, 513, 1], 264, 520
    E, R = len(M_list), sum(M_list)
    x = torch.randn(R, K).half().to(DEV)
    w = (torch.randn(E, 2 * I, K) * 0.1).half().to(DEV)
    M = _u32(M_list)
    h_ref = grouped_gemm(
        A=x, B=w, C=None, M_array=M, N_array=_u32([2 * I] * E), K_array=_u32([K] * E), output_shape=(R, 2 * I),
        is_A_transposed=False, is_B_transposed=True,
    )
    expect = O.grouped_gemm(x.cpu().float(), w.cpu().float(), M_list, [2 * I] * E, [K] * E, False, True).reshape(R, 2 * I)
    max_rel, frob_rel = rel_err(h_ref, expect)
    assert max_rel <= 2**-11 and frob_rel <= 2**-11
    h = torch.empty(R, 2 * I, dtype=torch.float16, device=DEV)
    act = torch.empty(R, I, dtype=torch.float16, device=DEV)
    grouped_gemm_swiglu_cuda(x, w, M, h, act)
    assert torch.equal(h, h_ref)
    assert torch.equal(act, swiglu_packed(h_ref))


def test_weight_gradient_layout_with_shuffled_ragged_reduction_lengths():
    # TN with a different reduction length per group, in no particular order, zeros included: the kernel orders the
    # groups by cost internally, the results must not depend on that
    g = torch.Generator().manual_seed(3)
    K_list = [0, 8, 4000, 64, 0, 1032, 72, 8, 2048, 136, 520, 8, 264, 1000, 0, 200] * 3
    E, M, N = len(K_list), 264, 520
    A, B = _integer_operands([M] * E, [N] * E, K_list, True, False, seed=13)
    expect = O.grouped_gemm(A, B, [M] * E, [N] * E, K_list, True, False)
    got = grouped_gemm(
        A=A.to(DEV), B=B.to(DEV), C=None, M_array=_u32([M] * E), N_array=_u32([N] * E), K_array=_u32(K_list),
        output_shape=(E * M * N,), is_A_transposed=True, is_B_transposed=False,
    )
    assert float((got.cpu().float() - expect.float()).abs().max()) == 0


@pytest.mark.parametrize("tA,tB", [(False, True), (True, False)])
def test_maximum_group_count(tA, tB):
    # 1024 groups (the limit), sizes that vary per group in every dimension, many empty
    g = torch.Generator().manual_seed(21)
    E = 1024
    M_list = (torch.randint(0, 5, (E,), generator=g) * 8).tolist()
    N_list = (torch.randint(1, 4, (E,), generator=g) * 8).tolist()
    K_list = (torch.randint(0, 20, (E,), generator=g) * 8).tolist()
    A, B = _integer_operands(M_list, N_list, K_list, tA, tB, seed=22)
    expect = O.grouped_gemm(A, B, M_list, N_list, K_list, tA, tB)
    got = grouped_gemm(
        A=A.to(DEV), B=B.to(DEV), C=None, M_array=_u32(M_list), N_array=_u32(N_list), K_array=_u32(K_list),
        output_shape=(sum(m * n for m, n in zip(M_list, N_list)),), is_A_transposed=tA, is_B_transposed=tB,
    )
    assert float((got.cpu().float() - expect.float()).abs().max()) == 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_groups_without_a_reduction_dimension_and_empty_outputs(dtype):
    # K_e == 0 for every group: both operands are empty tensors, the output is all zeros (found by a wider run of the
    # seeded random problems below: the wrapper used to hand the empty operand's NULL address to the entry point)
    M_list, N_list, K_list = [5, 0, 300], [16, 16, 16], [0, 0, 0]
    empty = torch.empty(0, dtype=dtype, device=DEV)
    got = grouped_gemm(
        A=empty, B=empty, C=None, M_array=_u32(M_list), N_array=_u32(N_list), K_array=_u32(K_list),
        output_shape=(305 * 16,), is_A_transposed=False, is_B_transposed=True,
    )
    assert got.shape == (305 * 16,) and float(got.float().abs().max()) == 0.0
    # no output at all (every group has M_e == 0): nothing to do
    none = grouped_gemm(
        A=empty, B=torch.ones(3 * 16 * 8, dtype=dtype, device=DEV), C=None, M_array=_u32([0, 0, 0]),
        N_array=_u32(N_list), K_array=_u32([8, 8, 8]), output_shape=(0,), is_A_transposed=False, is_B_transposed=True,
    )
    assert none.numel() == 0


@pytest.mark.parametrize("seed", [0, 1, 2, 3, 4, 5, 103])
def test_random_problem_shapes(seed):
    # seeded random problems: every layout, group counts 1..40, ragged / empty / one-row groups, reduction lengths from 0
    # to 17 K steps (even and odd step counts, partial last step), sizes off the 8-element grid now and then (scalar
    # path). Integer operands, so the fp32 sums are exact in any order and the bf16 result must match bit for bit.
    g = torch.Generator().manual_seed(1000 + seed)

    def draw(hi, grid):
        v = int(torch.randint(0, hi + 1, (1,), generator=g))
        return v if int(torch.randint(0, 8, (1,), generator=g)) == 0 and not grid else (v // 8) * 8

    for _ in range(6):
        tA, tB = bool(torch.randint(0, 2, (1,), generator=g)), bool(torch.randint(0, 2, (1,), generator=g))
        E = int(torch.randint(1, 41, (1,), generator=g))
        same_nk = bool(torch.randint(0, 2, (1,), generator=g))
        N0, K0 = max(8, draw(600, True)), draw(1100, True)
        M_list = [draw(700, False) for _ in range(E)]
        N_list = [N0 if same_nk else max(1, draw(600, False)) for _ in range(E)]
        K_list = [K0 if same_nk else draw(1100, False) for _ in range(E)]
        As, Bs, Ds = [], [], []
        for M, N, K in zip(M_list, N_list, K_list):
            a = torch.randint(-4, 5, (K, M) if tA else (M, K), generator=g).to(torch.bfloat16).to(DEV)
            b = torch.randint(-4, 5, (N, K) if tB else (K, N), generator=g).to(torch.bfloat16).to(DEV)
            As.append(a.reshape(-1))
            Bs.append(b.reshape(-1))
            Ds.append(((a.T if tA else a).float() @ (b.T if tB else b).float()).to(torch.bfloat16).reshape(-1))
        total = sum(m * n for m, n in zip(M_list, N_list))
        if total == 0:
            continue
        got = grouped_gemm(
            A=torch.cat(As), B=torch.cat(Bs), C=None, M_array=_u32(M_list), N_array=_u32(N_list), K_array=_u32(K_list),
            output_shape=(total,), is_A_transposed=tA, is_B_transposed=tB,
        )
        diff = float((got.float() - torch.cat(Ds).float()).abs().max())
        assert diff == 0, f"tA={tA} tB={tB} M={M_list} N={N_list} K={K_list}: max |diff| = {diff}"


@pytest.mark.parametrize("tA,tB", [(False, True), (False, False), (True, False)])
def test_random_problems_with_several_tiles_per_workgroup(tA, tB):
    # more tiles than workgroups, so every workgroup walks through tiles of different groups with different reduction
    # lengths (and reaches the next tile's first loads before it has stored the previous one)
    g = torch.Generator().manual_seed(77 + 2 * tA + tB)
    E = 24
    M_list = [int(v) * 8 for v in torch.randint(0, 1000, (E,), generator=g)]
    N_list = [int(v) * 8 for v in torch.randint(20, 130, (E,), generator=g)]
    K_list = [int(v) * 8 for v in torch.randint(0, 160, (E,), generator=g)]
    M_list[3], K_list[5] = 0, 0
    As, Bs, Ds = [], [], []
    for M, N, K in zip(M_list, N_list, K_list):
        a = torch.randint(-4, 5, (K, M) if tA else (M, K), generator=g).to(torch.bfloat16).to(DEV)
        b = torch.randint(-4, 5, (N, K) if tB else (K, N), generator=g).to(torch.bfloat16).to(DEV)
        As.append(a.reshape(-1))
        Bs.append(b.reshape(-1))
        Ds.append(((a.T if tA else a).float() @ (b.T if tB else b).float()).to(torch.bfloat16).reshape(-1))
    tiles = sum(-(-m // 256) * -(-n // 256) for m, n in zip(M_list, N_list))
    assert tiles > 3 * 256
    got = grouped_gemm(
        A=torch.cat(As), B=torch.cat(Bs), C=None, M_array=_u32(M_list), N_array=_u32(N_list), K_array=_u32(K_list),
        output_shape=(sum(m * n for m, n in zip(M_list, N_list)),), is_A_transposed=tA, is_B_transposed=tB,
    )
    assert float((got.float() - torch.cat(Ds).float()).abs().max()) == 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("layout", ["NT", "NN", "TN", "TT"])
def test_known_answer_fixture(layout, dtype):
    # tests/golden/grouped_gemm_kat.npz: int64 products of integer operands in [-8, 8] (four ragged groups, one empty);
    # every partial sum is an integer below 2^24, so the kernel's result is the stored product rounded once to the dtype
    import os

    import numpy as np
    from golden.make_golden import kat_problem

    fx = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "grouped_gemm_kat.npz"))
    M, N, K, tA, tB, As, Bs = kat_problem(layout)
    A = torch.from_numpy(np.concatenate([a.reshape(-1) for a in As])).to(dtype).to(DEV)
    B = torch.from_numpy(np.concatenate([b.reshape(-1) for b in Bs])).to(dtype).to(DEV)
    got = grouped_gemm(
        A=A, B=B, C=None, M_array=_u32(M), N_array=_u32(N), K_array=_u32(K),
        output_shape=(sum(m * n for m, n in zip(M, N)),), is_A_transposed=tA, is_B_transposed=tB,
    )
    assert got.dtype == dtype and torch.equal(got.cpu(), torch.from_numpy(fx[layout]).float().to(dtype))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("tB", [True, False])
@pytest.mark.parametrize("K", [192, 256, 320, 1000, 2112, 4096])  # 3, 4, 5, 16, 33, 64 K steps: every phase of the three-stage loop
def test_groups_of_few_rows_with_long_reductions(K, tB, dtype):
    # groups of at most 64 rows (batches of a few tokens per expert) run a K loop of their own with three LDS stages;
    # groups of 65 and 300 rows beside them take the usual loop. Integer operands in [-2, 2]: every partial sum is an
    # integer far below 2^24, so the kernel's result is the exact (int64) product rounded once to the dtype
    M_list, N = [1, 8, 33, 64, 0, 65, 17, 300, 64, 5], 328
    E = len(M_list)
    g = torch.Generator().manual_seed(K)
    As = [torch.randint(-2, 3, (m, K), generator=g) for m in M_list]
    Bs = [torch.randint(-2, 3, (N, K) if tB else (K, N), generator=g) for _ in M_list]
    A = torch.cat([a.reshape(-1) for a in As]).to(dtype).to(DEV)
    B = torch.cat([b.reshape(-1) for b in Bs]).to(dtype).to(DEV)
    got = grouped_gemm(
        A=A, B=B, C=None, M_array=_u32(M_list), N_array=_u32([N] * E), K_array=_u32([K] * E),
        output_shape=(sum(M_list) * N,), is_A_transposed=False, is_B_transposed=tB,
    )
    expect = torch.cat([(a @ (b.T if tB else b)).reshape(-1) for a, b in zip(As, Bs)]).float().to(dtype)  # int64 products
    assert torch.equal(got.cpu(), expect)


@pytest.mark.parametrize("K", [192, 1000, 4096])
def test_fused_swiglu_on_groups_of_few_rows(K):
    # the same for the fused epilogue: bit-identical to the plain GEMM followed by swiglu_packed
    M_list, I = [3, 64, 0, 40, 200, 64, 1], 136
    E, R = len(M_list), sum(M_list)
    g = torch.Generator().manual_seed(K + 1)
    x = (torch.randn(R, K, generator=g) * 0.5).bfloat16().to(DEV)
    w = (torch.randn(E, 2 * I, K, generator=g) * 0.05).bfloat16().to(DEV)
    h = torch.empty(R, 2 * I, dtype=torch.bfloat16, device=DEV)
    act = torch.empty(R, I, dtype=torch.bfloat16, device=DEV)
    grouped_gemm_swiglu_cuda(x, w, _u32(M_list), h, act)
    h_plain = grouped_gemm(
        A=x, B=w, C=None, M_array=_u32(M_list), N_array=_u32([2 * I] * E), K_array=_u32([K] * E),
        output_shape=(R, 2 * I), is_A_transposed=False, is_B_transposed=True,
    )
    assert torch.equal(h, h_plain) and torch.equal(act, swiglu_packed(h_plain))
    expect = torch.cat([xe.float() @ w[e].float().T for e, xe in enumerate(x.split(M_list))])
    assert float((h.float() - expect).abs().max()) <= 2**-8 * float(expect.abs().max())


def _exact_nt(x, w, M_list):
    """h_e = x_e @ w_e^T in float64 on the CPU (exact for small integers), rows of all groups back to back"""
    xs = x.cpu().double().split(M_list)
    return torch.cat([xs[e] @ w[e].cpu().double().T for e in range(len(M_list))])


def _small_group_case(M_list, N, K, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    E, R = len(M_list), sum(M_list)
    x = torch.randint(-3, 4, (R, K), generator=g).to(dtype).to(DEV)
    w = torch.randint(-3, 4, (E, N, K), generator=g).to(dtype).to(DEV)
    return x, w, _u32(M_list), E, R


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("K", [64, 192, 1000])
def test_half_width_tiles_many_small_groups(dtype, K):
    # Launches made of groups of at most 64 rows only, whose last round of full-width tiles would be at most half full, run
    # column tiles of half the width: 96 groups x 4 full-width tiles = 384 tiles = 1.5 rounds of 256 workgroups become 768
    # half-width tiles, several rounds, several per group, the last one of every group partial (1000 = 7 * 128 + 104).
    # Integers in [-3, 3]: |sum| <= 9000, exact in fp32 and, after rounding, compared as rounded values.
    M_list = [1 + (7 * e) % 64 for e in range(96)]
    N = 1000
    x, w, M, E, R = _small_group_case(M_list, N, K, dtype, seed=K)
    got = grouped_gemm(A=x, B=w, C=None, M_array=M, N_array=_u32([N] * E), K_array=_u32([K] * E), output_shape=(R, N),
                       is_A_transposed=False, is_B_transposed=True)
    expect = _exact_nt(x, w, M_list).to(dtype)
    assert torch.equal(got.cpu(), expect)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("K", [64, 192, 1000])
def test_half_width_tiles_fused_swiglu(dtype, K):
    # the same launch shape through the fused epilogue: I = 520 -> 5 tiles of 128 + 128 columns per group at full width
    # (480 tiles), 9 per group at half width, the last one 8 columns wide
    M_list = [1 + (5 * e) % 64 for e in range(96)]
    inter = 520
    x, w, M, E, R = _small_group_case(M_list, 2 * inter, K, dtype, seed=K + 1)
    h = torch.empty(R, 2 * inter, dtype=dtype, device=DEV)
    act = torch.empty(R, inter, dtype=dtype, device=DEV)
    grouped_gemm_swiglu_cuda(x, w, M, h, act)
    assert torch.equal(h.cpu(), _exact_nt(x, w, M_list).to(dtype))
    assert torch.equal(act, swiglu_packed(h))
    act_only = torch.empty_like(act)
    grouped_gemm_swiglu_cuda(x, w, M, None, act_only)
    assert torch.equal(act_only, act)


@pytest.mark.parametrize("fused", [False, True])
def test_half_width_decision_boundaries(fused):
    # The width is decided per launch from the tile counts and the number of workgroups (one per compute unit). Launches
    # just on either side of both thresholds: small groups only (half width while twice the tiles need at most 1.8 times
    # the rounds: groups = units / 2 and units / 2 + 1, one tile each), and small groups beside a large one (half width
    # while all tiles fill at most half of the workgroups).
    from fma import _lib

    units = _lib.load().fma_num_compute_units()
    assert units >= 8
    K, N = 192, 256
    cases = [[16] * (units // 2), [16] * (units // 2 + 1), [300] + [16] * (units // 2 - 2), [300] + [16] * (units // 2 - 1)]
    for i, M_list in enumerate(cases):
        x, w, M, E, R = _small_group_case(M_list, 2 * N if fused else N, K, torch.bfloat16, seed=40 + i)
        expect = _exact_nt(x, w, M_list).to(torch.bfloat16)
        if fused:
            h = torch.empty(R, 2 * N, dtype=torch.bfloat16, device=DEV)
            act = torch.empty(R, N, dtype=torch.bfloat16, device=DEV)
            grouped_gemm_swiglu_cuda(x, w, M, h, act)
            assert torch.equal(h.cpu(), expect), f"case {i}"
            assert torch.equal(act, swiglu_packed(h)), f"case {i}"
        else:
            got = grouped_gemm(A=x, B=w, C=None, M_array=M, N_array=_u32([N] * E), K_array=_u32([K] * E),
                               output_shape=(R, N), is_A_transposed=False, is_B_transposed=True)
            assert torch.equal(got.cpu(), expect), f"case {i}"
