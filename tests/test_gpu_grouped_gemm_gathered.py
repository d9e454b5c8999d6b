"""GPU parity of fma_grouped_gemm_gathered and fma_grouped_gemm_gathered_wgrad (the forward expert product and the weight
gradient with the gather of the routed rows inside the operand load) against fma_gather_rows followed by the entry points
that take packed rows: the same bits, for the plain and the fused-SwiGLU epilogue, with and without a bias; the weight
gradient also against a float64 product of the same rows."""

import pytest
import torch

from fma import _lib, swiglu_packed
from fma.modules.moe.cuda_implementation import (
    gather_rows_cuda,
    grouped_gemm_gathered_cuda,
    grouped_gemm_gathered_wgrad_cuda,
    grouped_gemm_ragged_cuda,
    grouped_gemm_swiglu_cuda,
)

from gpu_util import DEV

pytestmark = pytest.mark.gpu


def _u32(values):
    return torch.tensor(values, dtype=torch.int64).to(torch.uint32).to(DEV)


def _inputs(counts, T, K, N, divisor, dtype, seed):
    g = torch.Generator(device=DEV).manual_seed(seed)
    R, E = sum(counts), len(counts)
    x = torch.randn(T, K, device=DEV, generator=g).to(dtype)
    w = (torch.randn(E, N, K, device=DEV, generator=g) * 0.1).to(dtype)
    bias = torch.randn(E, N, device=DEV, generator=g).to(dtype)
    row_index = torch.randint(0, T * divisor, (R,), device=DEV, generator=g, dtype=torch.int32)
    xg = torch.empty(R, K, device=DEV, dtype=dtype)
    if R:
        gather_rows_cuda(x, row_index, divisor, xg)
    return x, w, bias, row_index, xg, _u32(counts)


CASES = [
    # rows per expert, T, K, N (plain) or 2 I (swiglu), divisor
    ([2048 + 8 * (e % 7) for e in range(24)], 4096, 512, 1024, 2),  # every workgroup streams through several tiles
    ([1500, 0, 264, 8, 3000, 40, 777 * 8], 700, 192, 768, 3),  # 3 K steps, thin and empty groups between
    ([520] * 40, 2000, 64, 512, 1),  # one K step per tile: both load slots of every tile belong to the next
    ([300, 5000, 16, 16, 16, 2000], 997, 1088, 256, 6),  # 17 K steps; groups of 16 rows run the three-stage loop
    ([1000, 1003, 2000], 5000, 72, 272, 8),  # a partial last K step; rows not a multiple of 8; a last column tile of 16
    ([40] * 64, 333, 136, 144, 64),  # half-width tiles
    ([1], 1, 8, 16, 1),
]


@pytest.mark.parametrize("with_bias", [False, True])
@pytest.mark.parametrize("counts,T,K,N,divisor", CASES)
def test_plain_epilogue(counts, T, K, N, divisor, with_bias):
    x, w, bias, row_index, xg, M = _inputs(counts, T, K, N, divisor, torch.bfloat16, seed=K + N)
    R = sum(counts)
    expect = torch.full((R, N), 7.0, dtype=torch.bfloat16, device=DEV)
    grouped_gemm_ragged_cuda(xg, w, expect, M, False, 0, N, K, False, True, bias if with_bias else None)
    got = torch.full((R, N), 7.0, dtype=torch.bfloat16, device=DEV)
    grouped_gemm_gathered_cuda(x, row_index, divisor, w, bias if with_bias else None, M, got, None)
    assert torch.equal(got, expect)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("with_bias", [False, True])
@pytest.mark.parametrize("counts,T,K,N,divisor", CASES)
def test_swiglu_epilogue(counts, T, K, N, divisor, with_bias, dtype):
    x, w, bias, row_index, xg, M = _inputs(counts, T, K, N, divisor, dtype, seed=K + N + 1)
    R = sum(counts)
    b = bias if with_bias else None
    h_ref = torch.full((R, N), 7.0, dtype=dtype, device=DEV)
    act_ref = torch.full((R, N // 2), 7.0, dtype=dtype, device=DEV)
    grouped_gemm_swiglu_cuda(xg, w, M, h_ref, act_ref, b)
    h = torch.full((R, N), 7.0, dtype=dtype, device=DEV)
    act = torch.full((R, N // 2), 7.0, dtype=dtype, device=DEV)
    grouped_gemm_gathered_cuda(x, row_index, divisor, w, b, M, h, act)
    assert torch.equal(h, h_ref) and torch.equal(act, act_ref)
    assert torch.equal(act, swiglu_packed(h))
    act_only = torch.full((R, N // 2), 7.0, dtype=dtype, device=DEV)
    grouped_gemm_gathered_cuda(x, row_index, divisor, w, b, M, None, act_only)
    assert torch.equal(act_only, act_ref)


@pytest.mark.parametrize("counts,T,K,N,divisor", [CASES[0], CASES[3], CASES[5]])
def test_index_entries_that_name_no_row_read_as_zero_rows(counts, T, K, N, divisor):
    # negative entries and entries past the last row of x: their rows of the operand are zeros, so the output row is the
    # bias (plain epilogue); every other row as before
    x, w, bias, row_index, xg, M = _inputs(counts, T, K, N, divisor, torch.bfloat16, seed=5)
    R = sum(counts)
    bad = torch.arange(R, device=DEV) % 7 == 3
    broken = row_index.clone()
    broken[bad & (torch.arange(R, device=DEV) % 2 == 0)] = -5
    broken[bad & (torch.arange(R, device=DEV) % 2 == 1)] = T * divisor + 11
    xg_zeroed = xg.clone()
    xg_zeroed[bad] = 0
    expect = torch.full((R, N), 7.0, dtype=torch.bfloat16, device=DEV)
    grouped_gemm_ragged_cuda(xg_zeroed, w, expect, M, False, 0, N, K, False, True, bias)
    got = torch.full((R, N), 7.0, dtype=torch.bfloat16, device=DEV)
    grouped_gemm_gathered_cuda(x, broken, divisor, w, bias, M, got, None)
    assert torch.equal(got, expect)


def test_repeated_launches_and_the_routing_order():
    # the layer's use: row_index = the stable routing order of T * k slots, divisor = k; three launches into fresh buffers
    T, k, E, K, N = 3000, 2, 8, 256, 512
    g = torch.Generator(device=DEV).manual_seed(5)
    ids = torch.randint(0, E, (T * k,), device=DEV, generator=g)
    order = torch.sort(ids, stable=True).indices.to(torch.int32)
    counts = torch.bincount(ids, minlength=E).tolist()
    x = torch.randn(T, K, device=DEV, generator=g).bfloat16()
    w = (torch.randn(E, N, K, device=DEV, generator=g) * 0.1).bfloat16()
    xg = x[(order // k).long()].contiguous()
    expect = torch.empty(T * k, N, dtype=torch.bfloat16, device=DEV)
    grouped_gemm_ragged_cuda(xg, w, expect, _u32(counts), False, 0, N, K, False, True)
    for _ in range(3):
        got = torch.full((T * k, N), 7.0, dtype=torch.bfloat16, device=DEV)
        grouped_gemm_gathered_cuda(x, order, k, w, None, _u32(counts), got, None)
        assert torch.equal(got, expect)


def test_argument_validation():
    lib = _lib.load()
    p = torch.zeros(4096, dtype=torch.bfloat16, device=DEV).data_ptr()
    m = _u32([8]).data_ptr()
    call = lib.fma_grouped_gemm_gathered
    assert call(p, 8, None, 1, p, None, p, None, m, 1, 16, 16, 0, _lib.FMA_BF16, None) == -1  # no row index
    assert call(p, 8, p, 0, p, None, p, None, m, 1, 16, 16, 0, _lib.FMA_BF16, None) == -3  # divisor
    assert call(p, 8, p, 1, p, None, p, None, m, 1, 12, 16, 0, _lib.FMA_BF16, None) == -3  # N % 8
    assert call(p, 8, p, 1, p, None, p, None, m, 1, 16, 12, 0, _lib.FMA_BF16, None) == -3  # K % 8
    assert call(p, 1 << 27, p, 1, p, None, p, None, m, 1, 16, 16, 0, _lib.FMA_BF16, None) == -8  # x of 4 GiB
    assert call(p, 8, p, 1, p, None, None, None, m, 1, 16, 16, 0, _lib.FMA_BF16, None) == -1  # no output
    assert call(p, 8, p, 1, p, None, p, None, m, 1, 16, 16, 0, _lib.FMA_F32, None) != 0  # 16-bit types only
    assert call(p, 8, p, 1, p, None, p, None, m, 0, 16, 16, 0, _lib.FMA_BF16, None) == 0  # no groups


WGRAD_CASES = [
    # rows per expert, T, N (rows of the gradient's output, = out features), K (= in features, width of x), divisor
    ([2048 + 8 * (e % 7) for e in range(8)], 4096, 512, 1024, 2),  # long reductions: every tile streams into the next
    ([1500, 0, 263, 7, 3001, 40, 777], 700, 768, 192, 3),  # reductions of any length, empty groups, K one partial tile
    ([520] * 40, 2000, 256, 512, 1),  # 9 K steps per tile (the last one partial), many tiles per workgroup
    ([64, 63, 65, 128, 129, 191, 192, 193, 1, 2], 50, 256, 512, 4),  # 1 to 4 K steps: tiles that start cold
    ([300, 5000, 16, 16, 16, 2000], 997, 264, 1088, 6),  # N and K with partial tiles
    ([0, 0, 5], 9, 256, 256, 1),
    ([0, 0, 0], 9, 256, 256, 1),
    ([(37 * e) % 211 for e in range(300)], 1234, 264, 520, 5),  # many short groups: every tile starts cold; partial tiles both ways
    ([193 + (e % 3) * 64 for e in range(40)], 4000, 512, 256, 2),  # 4 or 5 K steps: streamed tiles of the shortest kind
]


def _wgrad_inputs(counts, T, N, K, divisor, dtype, seed, spoil=False):
    g = torch.Generator(device=DEV).manual_seed(seed)
    R, E = sum(counts), len(counts)
    x = torch.randn(T, K, device=DEV, generator=g).to(dtype)
    dy = torch.randn(R, N, device=DEV, generator=g).to(dtype)
    row_index = torch.randint(0, T * divisor, (R,), device=DEV, generator=g, dtype=torch.int32)
    if spoil and R > 10:
        row_index[3] = -5
        row_index[R // 2] = T * divisor + 7
        row_index[R - 1] = -(2**31)
    xg = torch.zeros(R, K, device=DEV, dtype=dtype)
    if R:
        src = torch.div(row_index.long(), divisor, rounding_mode="floor")
        ok = (row_index >= 0) & (src < T)
        xg[ok] = x[src[ok]]
    return x, dy, row_index, xg, _u32(counts)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("spoil", [False, True])
@pytest.mark.parametrize("counts,T,N,K,divisor", WGRAD_CASES)
def test_weight_gradient_gathers_its_reduction_rows(counts, T, N, K, divisor, spoil, dtype):
    x, dy, row_index, xg, sizes = _wgrad_inputs(counts, T, N, K, divisor, dtype, seed=N + K + divisor, spoil=spoil)
    E = len(counts)
    # the packed kernel on an explicit copy of the rows (entries that name no row: rows of zeros): the same bits
    expect = torch.full((E, N, K), 7.0, dtype=dtype, device=DEV)
    grouped_gemm_ragged_cuda(dy, xg, expect, sizes, True, N, K, 0, True, False)
    got = torch.full((E, N, K), 7.0, dtype=dtype, device=DEV)
    grouped_gemm_gathered_wgrad_cuda(dy, x, row_index, divisor, sizes, got)
    assert torch.equal(got, expect)
    # and the product itself, in float64 (one rounding of an fp32-accumulated sum: 2^-8 relative for bf16, 2^-11 for fp16,
    # of the largest element of the group's gradient, plus the accumulation's own error)
    start = 0
    for e, m in enumerate(counts):
        ref = dy[start : start + m].double().T @ xg[start : start + m].double()
        tol = (2.0**-8 if dtype == torch.bfloat16 else 2.0**-11) * float(ref.abs().max()) + 1e-6 * m
        assert float((got[e].double() - ref).abs().max()) <= tol, f"expert {e}"
        start += m


def test_weight_gradient_scaled_by_alpha():
    counts, T, N, K, divisor = [700, 0, 129], 300, 264, 512, 2
    x, dy, row_index, xg, sizes = _wgrad_inputs(counts, T, N, K, divisor, torch.bfloat16, seed=9)
    lib, E = _lib.load(), len(counts)
    stream = torch.cuda.current_stream().cuda_stream
    expect = torch.empty(E, N, K, dtype=torch.bfloat16, device=DEV)
    got = torch.empty(E, N, K, dtype=torch.bfloat16, device=DEV)
    rc = lib.fma_grouped_gemm_ragged(dy.data_ptr(), xg.data_ptr(), expect.data_ptr(), sizes.data_ptr(), None, E, _lib.FMA_VARY_K,
                                     N, K, 0, 1, 0, -0.375, _lib.FMA_BF16, stream)
    _lib.check(rc, "fma_grouped_gemm_ragged")
    rc = lib.fma_grouped_gemm_gathered_wgrad(dy.data_ptr(), x.data_ptr(), T, row_index.data_ptr(), divisor, got.data_ptr(),
                                             sizes.data_ptr(), E, N, K, -0.375, _lib.FMA_BF16, stream)
    _lib.check(rc, "fma_grouped_gemm_gathered_wgrad")
    assert torch.equal(got, expect) and bool((got[1] == 0).all()) and float(got[0].abs().max()) > 0


def test_weight_gradient_argument_validation():
    lib = _lib.load()
    call = lib.fma_grouped_gemm_gathered_wgrad
    buf = torch.zeros(1 << 16, dtype=torch.bfloat16, device=DEV)
    idx = torch.zeros(64, dtype=torch.int32, device=DEV)
    k = _u32([8])
    p, i, s = buf.data_ptr(), idx.data_ptr(), k.data_ptr()
    bf = _lib.FMA_BF16
    assert call(p, p, 8, i, 1, p, s, 1, 16, 16, 1.0, bf, None) == 0
    torch.cuda.synchronize()
    assert call(p, p, 8, i, 1, p, s, 1, 12, 16, 1.0, bf, None) != 0  # M not a multiple of 8
    assert call(p, p, 8, i, 1, p, s, 1, 16, 20, 1.0, bf, None) != 0  # N not a multiple of 8
    assert call(p, p, 8, i, 0, p, s, 1, 16, 16, 1.0, bf, None) != 0  # divisor
    assert call(p, p, 0, i, 1, p, s, 1, 16, 16, 1.0, bf, None) != 0  # x without rows
    assert call(p, p, 1 << 28, i, 1, p, s, 1, 16, 16, 1.0, bf, None) != 0  # x of 2 GiB or more
    assert call(p, p, 8, None, 1, p, s, 1, 16, 16, 1.0, bf, None) != 0  # no row_index
    assert call(p, p, 8, i, 1, p, s, 1, 16, 16, 1.0, _lib.FMA_F32, None) != 0  # 16-bit types only
    assert call(p + 2, p, 8, i, 1, p, s, 1, 16, 16, 1.0, bf, None) != 0  # misaligned
    assert call(p, p, 8, i, 1, p, s, 0, 16, 16, 1.0, bf, None) == 0  # no groups
    assert "grouped_gemm_gathered_wgrad" in lib.fma_last_error_string().decode()


@pytest.mark.parametrize("act_name,add_bias", [("swiglu", False), ("swiglu", True), ("gelu", True), ("glu", False)])
def test_layer_with_the_gather_inside_the_first_projection(act_name, add_bias):
    # the layer with and without the grouped copy of the tokens: the same bits in the output and in every gradient
    import torch.nn as nn

    from fma import KernelBackend, MoE

    torch.manual_seed(3)
    E, k, H, I, T = 8, 2, 256, 512, 300
    is_glu = act_name != "gelu"
    act = {"swiglu": swiglu_packed, "glu": nn.GLU(), "gelu": nn.GELU(approximate="tanh")}[act_name]
    moe = MoE(E, k, H, I, act, is_glu, add_bias, 0.02).to(torch.bfloat16).to(DEV)
    if add_bias:
        with torch.no_grad():
            moe.c_fc.bias.normal_(0, 0.5)
            moe.c_proj.bias.normal_(0, 0.5)
    x = torch.randn(T, H, device=DEV).bfloat16()
    dy = torch.randn(T, H, device=DEV).bfloat16()
    results = []
    for gather in (False, True):
        moe.gather_in_gemm = gather
        moe.zero_grad()
        xi = x.clone().requires_grad_()
        y, _ = moe(xi, kernel_backend=KernelBackend.cuda)
        y.backward(dy)
        results.append([y.detach(), xi.grad] + [p.grad.clone() for p in moe.parameters()])
    for a, b in zip(*results):
        assert torch.equal(a, b)


def test_when_the_layer_writes_a_grouped_copy_of_the_tokens(monkeypatch):
    # a narrow first projection gathers by itself, in its forward and in its weight gradient: no row-movement pass in
    # front of it, with or without a backward; a wide one reads a grouped copy of the tokens
    from fma import KernelBackend, MoE
    from fma.modules.moe import cuda_implementation as ci

    torch.manual_seed(4)
    calls = []
    real = ci.dispatch_rows_cuda
    monkeypatch.setattr(ci, "dispatch_rows_cuda", lambda *a: (calls.append(1), real(*a))[1])
    x = torch.randn(100, 256, device=DEV).bfloat16()
    moe = MoE(8, 2, 256, 512, swiglu_packed, True, False, 0.02).to(torch.bfloat16).to(DEV)
    xi = x.clone().requires_grad_()
    y_train, _ = moe(xi, kernel_backend=KernelBackend.cuda)
    y_train.sum().backward()
    with torch.no_grad():
        y_eval, _ = moe(x, kernel_backend=KernelBackend.cuda)
    assert calls == [] and torch.equal(y_eval, y_train.detach())
    assert xi.grad is not None and moe.c_fc.weight.grad is not None
    wide = MoE(2, 2, 256, 3200, swiglu_packed, True, False, 0.02).to(torch.bfloat16).to(DEV)
    wide(x.clone().requires_grad_(), kernel_backend=KernelBackend.cuda)
    assert calls == [1]
