"""GPU parity of fma_grouped_gemm_ragged (groups that differ in one dimension, operand loads streamed across tile
boundaries): exact on integer-valued operands against float64 products, and bit-identical to fma_grouped_gemm with the
other two dimensions spelled out per group. The cases are chosen to walk every kind of tile boundary: several tiles per
workgroup in a row, odd and even numbers of K steps, tiles with few rows, groups of at most 64 rows (their own K loop),
empty groups, groups without reduction, and groups that need the element-wise path in the middle of the sequence."""

import pytest
import torch

from fma import _lib, grouped_gemm

from gpu_util import DEV

pytestmark = pytest.mark.gpu


def _u32(values):
    return torch.tensor(values, dtype=torch.int64).to(torch.uint32).to(DEV)


def _ragged(A, B, sizes, vary_k, M, N, K, tA, tB, out_elems, alpha=1.0, bias=None):
    lib = _lib.load()
    out = torch.full((max(out_elems, 1),), 7.0, dtype=A.dtype, device=DEV)
    s = _u32(sizes)
    rc = lib.fma_grouped_gemm_ragged(
        A.data_ptr(), B.data_ptr(), out.data_ptr(), s.data_ptr(), _lib.ptr(bias), len(sizes),
        _lib.FMA_VARY_K if vary_k else _lib.FMA_VARY_M, M, N, K, int(tA), int(tB), alpha, _lib.dtype_code(A.dtype), torch.cuda.current_stream().cuda_stream,
    )
    assert rc == 0, lib.fma_last_error_string()
    torch.cuda.synchronize()
    return out[:out_elems]


def _case(sizes, vary_k, M, N, K, tA, tB, dtype, seed):
    """operands, the exact result (float64 on the GPU, rounded once) and the generic entry point's result"""
    g = torch.Generator(device=DEV).manual_seed(seed)
    Ms = [M] * len(sizes) if vary_k else sizes
    Ks = sizes if vary_k else [K] * len(sizes)
    As, Bs, Ds = [], [], []
    for m, k in zip(Ms, Ks):
        a = torch.randint(-3, 4, (k, m) if tA else (m, k), device=DEV, generator=g).to(dtype)
        b = torch.randint(-3, 4, (N, k) if tB else (k, N), device=DEV, generator=g).to(dtype)
        As.append(a.reshape(-1))
        Bs.append(b.reshape(-1))
        Ds.append(((a.T if tA else a).double() @ (b.T if tB else b).double()).to(dtype).reshape(-1))
    pad = torch.zeros(8, dtype=dtype, device=DEV)  # an operand may be empty: keep a valid address
    A, B, expect = torch.cat(As + [pad]), torch.cat(Bs + [pad]), torch.cat(Ds) if Ds else pad[:0]
    n_out = sum(m * N for m in Ms)
    generic = grouped_gemm(
        A=A, B=B, C=None, M_array=_u32(Ms), N_array=_u32([N] * len(sizes)), K_array=_u32(Ks), output_shape=(max(n_out, 1),),
        is_A_transposed=tA, is_B_transposed=tB,
    )[:n_out]
    return A, B, expect, generic, n_out


LAYOUTS = [(False, True), (False, False), (True, False), (True, True)]


@pytest.mark.parametrize("tA,tB", LAYOUTS)
@pytest.mark.parametrize(
    "sizes,N,K",
    [
        ([2048 + 8 * (e % 7) for e in range(24)], 1024, 512),  # 800 tiles: every workgroup streams through several, 8 K steps
        ([1500, 0, 264, 8, 3000, 40, 777 * 8], 768, 192),  # 3 K steps (a step of zeros appended), thin and empty groups between
        ([520] * 40, 512, 64),  # one K step per tile: both load slots of every tile belong to the next
        ([300, 5000, 16, 16, 16, 2000], 256, 1088),  # 17 K steps; groups of 16 rows run the three-stage loop in the middle
        ([1000, 1003, 2000], 264, 128),  # a group whose rows are not a multiple of 8: element-wise path where M is contiguous
    ],
)
def test_rows_vary(tA, tB, sizes, N, K):
    A, B, expect, generic, n_out = _case(sizes, False, 0, N, K, tA, tB, torch.bfloat16, seed=len(sizes) + N)
    got = _ragged(A, B, sizes, False, 0, N, K, tA, tB, n_out)
    assert torch.equal(got, expect), f"max diff {float((got.float() - expect.float()).abs().max())}"
    assert torch.equal(got, generic)


@pytest.mark.parametrize("tA,tB", LAYOUTS)
@pytest.mark.parametrize(
    "sizes,M,N",
    [
        ([512 + 64 * (e % 5) for e in range(20)], 1024, 768),  # weight-gradient shape: 8 to 12 K steps, 240 tiles... x 20 groups
        ([4096, 0, 72, 8, 1000, 0, 3000], 512, 1024),  # empty experts (exact zeros), ragged reduction lengths, odd step counts
        ([200] * 48, 768, 256),  # 4 K steps, the last one a quarter full; 144 tiles
    ],
)
def test_reduction_varies(tA, tB, sizes, M, N):
    A, B, expect, generic, n_out = _case(sizes, True, M, N, 0, tA, tB, torch.bfloat16, seed=len(sizes) + M)
    got = _ragged(A, B, sizes, True, M, N, 0, tA, tB, n_out)
    assert torch.equal(got, expect), f"max diff {float((got.float() - expect.float()).abs().max())}"
    assert torch.equal(got, generic)
    # groups without reduction are exact zeros (and are written: the buffer was filled with 7)
    off = 0
    for k in sizes:
        if k == 0:
            assert float(got[off:off + M * N].float().abs().max()) == 0.0
        off += M * N


@pytest.mark.parametrize("tA,tB", [(False, True), (True, False)])
def test_fp16_and_alpha(tA, tB):
    sizes, N, K = [700, 0, 1032, 24], 512, 320
    A, B, expect, generic, n_out = _case(sizes, False, 0, N, K, tA, tB, torch.float16, seed=3)
    got = _ragged(A, B, sizes, False, 0, N, K, tA, tB, n_out)
    assert torch.equal(got, expect) and torch.equal(got, generic)
    half = _ragged(A, B, sizes, False, 0, N, K, tA, tB, n_out, alpha=0.5)
    assert torch.equal(half.float(), (expect.double() * 0.5).to(torch.float16).float())


def test_many_groups_and_repeated_launches():
    # 1024 groups (the limit), most of them tiny, and the same launch three times into a fresh buffer
    sizes = [(37 * e) % 300 for e in range(1024)]
    N, K = 256, 128
    A, B, expect, generic, n_out = _case(sizes, False, 0, N, K, False, True, torch.bfloat16, seed=11)
    for _ in range(3):
        got = _ragged(A, B, sizes, False, 0, N, K, False, True, n_out)
        assert torch.equal(got, expect) and torch.equal(got, generic)


def test_argument_validation():
    lib = _lib.load()
    p = torch.zeros(64, dtype=torch.bfloat16, device=DEV).data_ptr()
    s = _u32([8]).data_ptr()
    assert lib.fma_grouped_gemm_ragged(p, p, p, s, None, 1, 2, 8, 8, 8, 0, 1, 1.0, _lib.FMA_BF16, None) == -3  # vary
    assert lib.fma_grouped_gemm_ragged(p, p, p, s, None, 1, 0, 8, 8, 8, 0, 1, 1.0, _lib.FMA_F32, None) != 0  # fp32: other entry
    assert lib.fma_grouped_gemm_ragged(p, p, p, s, None, 1025, 0, 8, 8, 8, 0, 1, 1.0, _lib.FMA_BF16, None) == -4
    assert lib.fma_grouped_gemm_ragged(p, p, None, s, None, 1, 0, 8, 8, 8, 0, 1, 1.0, _lib.FMA_BF16, None) == -1
    assert lib.fma_grouped_gemm_ragged(p, p + 2, p, s, None, 1, 0, 8, 8, 8, 0, 1, 1.0, _lib.FMA_BF16, None) == -6
    assert lib.fma_grouped_gemm_ragged(p, p, p, s, None, 0, 0, 8, 8, 8, 0, 1, 1.0, _lib.FMA_BF16, None) == 0  # no groups
