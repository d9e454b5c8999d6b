"""Tensors past 2^31 elements and 2^32 bytes (a long batch on a 288 GB device): every kernel's index arithmetic at
sizes where 32-bit offsets would wrap. Each op is checked exactly — against torch on integer-valued data where the
arithmetic is then exact, or against the same op run on row chunks small enough for 32-bit offsets — so a wrapped
offset anywhere shows up as a mismatch in the chunk it lands in. Peak device memory of one test is about 45 GB."""

import pytest
import torch

from fma import continuous_count, fused_residual_add_rmsnorm, grouped_gemm, swiglu_packed
from fma.modules.moe import cuda_implementation as C

from gpu_util import DEV

pytestmark = pytest.mark.gpu

BF16 = torch.bfloat16


def _u32(values):
    return torch.tensor(values, dtype=torch.int64).to(torch.uint32).to(DEV)


def _chunks(n, step):
    for a in range(0, n, step):
        yield a, min(n, a + step)


@pytest.fixture(autouse=True)
def _release_device_memory():
    yield
    torch.cuda.empty_cache()


def test_swiglu_packed_past_2_31_elements():
    R, N = 131080, 28672  # 3.76e9 elements in, 7.5e9 bytes
    x = torch.randn(R, N, device=DEV, dtype=BF16).requires_grad_()
    dy = torch.randn(R, N // 2, device=DEV, dtype=BF16)
    y = swiglu_packed(x)
    y.backward(dy)
    for a, b in _chunks(R, 16384):
        xc = x[a:b].detach().clone().requires_grad_()
        yc = swiglu_packed(xc)
        yc.backward(dy[a:b])
        assert torch.equal(yc, y[a:b]), f"forward, rows {a}.."
        assert torch.equal(xc.grad, x.grad[a:b]), f"backward, rows {a}.."


def test_grouped_gemm_with_groups_past_2_32_bytes():
    # the second group's rows of the big operand start 4.6e9 bytes into it
    M_list, N, K = [80008, 51064], 28672, 256
    g = torch.Generator(device=DEV).manual_seed(1)
    A = torch.randint(-8, 9, (sum(M_list), K), device=DEV, generator=g).to(BF16)
    B = torch.randint(-8, 9, (2, N, K), device=DEV, generator=g).to(BF16)
    D = grouped_gemm(
        A=A.reshape(-1), B=B.reshape(-1), C=None, M_array=_u32(M_list), N_array=_u32([N] * 2), K_array=_u32([K] * 2),
        output_shape=(sum(M_list) * N,), is_A_transposed=False, is_B_transposed=True,
    ).view(sum(M_list), N)
    row = 0
    for e, m in enumerate(M_list):
        for a, b in _chunks(m, 16384):
            # integer operands: sums below 2^24, one rounding to bf16 on both sides
            assert torch.equal(D[row + a : row + b], A[row + a : row + b] @ B[e].T), f"NT, group {e}, rows {a}.."
        row += m
    # the big tensor as the reduction-major operand of the weight-gradient form and as the row operand of the
    # input-gradient form (products of up to 80008 terms: compared in relative terms against fp32 matrix products)
    Dw = grouped_gemm(
        A=D.reshape(-1), B=A.reshape(-1), C=None, M_array=_u32([N] * 2), N_array=_u32([K] * 2), K_array=_u32(M_list),
        output_shape=(2 * N * K,), is_A_transposed=True, is_B_transposed=False,
    ).view(2, N, K)
    Dx = grouped_gemm(
        A=D.reshape(-1), B=B.reshape(-1), C=None, M_array=_u32(M_list), N_array=_u32([K] * 2), K_array=_u32([N] * 2),
        output_shape=(sum(M_list) * K,), is_A_transposed=False, is_B_transposed=False,
    ).view(sum(M_list), K)
    row = 0
    for e, m in enumerate(M_list):
        ref_w = D[row : row + m].float().T @ A[row : row + m].float()
        ref_x = D[row : row + m].float() @ B[e].float()
        assert float((Dw[e].float() - ref_w).abs().max()) <= 2**-7 * float(ref_w.abs().max()), f"TN, group {e}"
        assert float((Dx[row : row + m].float() - ref_x).abs().max()) <= 2**-7 * float(ref_x.abs().max()), f"NN, group {e}"
        row += m


def test_gathered_products_on_a_token_matrix_of_almost_2_31_bytes():
    # the gathered kernels address x with 32-bit byte offsets below 2^31: x as large as they admit, with most of the
    # routed rows taken from its last rows, and the dy operand of the weight gradient past 2^32 bytes
    T, H, N, k = 262143, 4096, 512, 2  # x: 2^31 - 8192 bytes
    counts = [40000, 8, 60000, 31064]
    R = sum(counts)
    g = torch.Generator(device=DEV).manual_seed(2)
    x = torch.randint(-8, 9, (T, H), device=DEV, generator=g).to(BF16)
    perm = torch.randint(T * k - 4096, T * k, (R,), device=DEV, generator=g, dtype=torch.int32)
    perm[::7] = torch.randint(0, T * k, (len(perm[::7]),), device=DEV, generator=g, dtype=torch.int32)
    perm[-1] = T * k - 1
    xg = x[perm.long() // k]
    sizes = _u32(counts)
    w = torch.randint(-8, 9, (len(counts), N, H), device=DEV, generator=g).to(BF16)
    expect = torch.empty(R, N, device=DEV, dtype=BF16)
    C.grouped_gemm_ragged_cuda(xg, w, expect, sizes, False, 0, N, H, False, True)
    got = torch.empty(R, N, device=DEV, dtype=BF16)
    C.grouped_gemm_gathered_cuda(x, perm, k, w, None, sizes, got, None)
    assert torch.equal(got, expect)
    del w, expect, got
    M = 32768  # dy: 131072 rows of 32768 elements, 8.6e9 bytes
    dy = torch.randint(-2, 3, (R, M), device=DEV, generator=g).to(BF16)
    dw_expect = torch.empty(len(counts), M, H, device=DEV, dtype=BF16)
    C.grouped_gemm_ragged_cuda(dy, xg, dw_expect, sizes, True, M, H, 0, True, False)
    dw = torch.empty(len(counts), M, H, device=DEV, dtype=BF16)
    C.grouped_gemm_gathered_wgrad_cuda(dy, x, perm, k, sizes, dw)
    assert torch.equal(dw, dw_expect)
    # integer operands, sums below 2^24: the small group's gradient is exact
    e0 = counts[0]
    ref = dy[e0 : e0 + 8].float().T @ xg[e0 : e0 + 8].float()
    assert torch.equal(dw[1].float(), ref)


def test_row_kernels_on_10_gb_of_grouped_rows():
    T, k, H, E = 300000, 4, 4096, 16  # 1.2M grouped rows of 8 KB
    R = T * k
    g = torch.Generator(device=DEV).manual_seed(2)
    x = torch.randint(-8, 9, (T, H), device=DEV, generator=g).to(BF16)
    selected = torch.randint(0, E, (T, k), device=DEV, generator=g)
    _, _, perm, eid, inv = C.build_routing_index(selected, E)
    order = torch.sort(selected.reshape(-1), stable=True)
    assert torch.equal(perm.long(), order.indices) and torch.equal(eid.long(), order.values)
    del order

    xg = torch.empty(R, H, device=DEV, dtype=BF16)
    C.gather_rows_cuda(x, perm, k, xg)
    for a, b in _chunks(R, 131072):
        assert torch.equal(xg[a:b], x[(perm[a:b] // k).long()]), f"gather, rows {a}.."
    xd = torch.empty(R, H, device=DEV, dtype=BF16)
    C.dispatch_rows_cuda(x, inv, k, xd)
    for a, b in _chunks(R, 131072):
        assert torch.equal(xd[a:b], xg[a:b]), f"dispatch, rows {a}.."
    del xd

    # small integers times powers of two: every sum is exact in fp32, so torch's order of additions does not matter
    gates = (2.0 ** torch.randint(-2, 2, (T, k), device=DEV, generator=g).float()).to(BF16)
    y = torch.empty(T, H, device=DEV, dtype=BF16)
    C.combine_cuda(xg, inv, gates, k, y)
    dy = torch.randint(-8, 9, (T, H), device=DEV, generator=g).to(BF16)
    d_o = torch.empty(R, H, device=DEV, dtype=BF16)
    d_gates = torch.empty(T, k, device=DEV, dtype=BF16)
    C.combine_backward_cuda(dy, xg, inv, gates, k, d_o, d_gates)
    for a, b in _chunks(T, 32768):
        idx = inv.view(T, k)[a:b].long().reshape(-1)
        rows = xg[idx].view(b - a, k, H).float()
        assert torch.equal(y[a:b], (rows * gates[a:b].float()[..., None]).sum(1).to(BF16)), f"combine, tokens {a}.."
        assert torch.equal(d_gates[a:b], (rows * dy[a:b].float()[:, None, :]).sum(-1).to(BF16)), f"gate gradient, tokens {a}.."
        expect = (dy[a:b].float()[:, None, :] * gates[a:b].float()[..., None]).to(BF16).view(-1, H)
        assert torch.equal(d_o[idx], expect), f"grouped-row gradient, tokens {a}.."


def test_residual_add_rmsnorm_past_2_32_bytes():
    B, H = 600000, 4096  # 4.9e9 bytes per tensor
    x = torch.randn(B, H, device=DEV, dtype=BF16).requires_grad_()
    r = torch.randn(B, H, device=DEV, dtype=BF16).requires_grad_()
    w = torch.randn(H, device=DEV, dtype=BF16).requires_grad_()
    dy = torch.randn(B, H, device=DEV, dtype=BF16)
    y, rr = fused_residual_add_rmsnorm(x, r, w, 1e-5, multiplier=0.5)
    torch.autograd.backward([y, rr], [dy, dy])
    w_sum = torch.zeros(H, device=DEV, dtype=torch.float64)
    for a, b in _chunks(B, 65536):
        xc, rc = x[a:b].detach().clone().requires_grad_(), r[a:b].detach().clone().requires_grad_()
        wc = w.detach().clone().requires_grad_()
        yc, rrc = fused_residual_add_rmsnorm(xc, rc, wc, 1e-5, multiplier=0.5)
        torch.autograd.backward([yc, rrc], [dy[a:b], dy[a:b]])
        assert torch.equal(yc, y[a:b]) and torch.equal(rrc, rr[a:b]), f"forward, rows {a}.."
        assert torch.equal(xc.grad, x.grad[a:b]) and torch.equal(rc.grad, r.grad[a:b]), f"backward, rows {a}.."
        w_sum += wc.grad.double()
    # the weight gradient sums over all rows: the chunks' bf16-rounded partial results add up to it within their rounding
    assert float((w.grad.double() - w_sum).abs().max()) <= 2e-2 * float(w_sum.abs().max())


def test_expert_bias_past_2_32_bytes():
    E, N, M_list = 4, 28672, [70000, 0, 50000, 30000]  # 8.6e9 bytes
    R = sum(M_list)
    y = torch.randn(R, N, device=DEV, dtype=BF16)
    bias = torch.randn(E, N, device=DEV, dtype=BF16)
    before = y.clone()
    C.expert_bias_add_cuda(y, bias, _u32(M_list))
    bias_grad = torch.empty(E, N, device=DEV, dtype=BF16)
    C.expert_bias_grad_cuda(before, _u32(M_list), bias_grad)
    row = 0
    for e, m in enumerate(M_list):
        for a, b in _chunks(m, 16384):
            assert torch.equal(y[row + a : row + b], before[row + a : row + b] + bias[e]), f"bias add, group {e}, rows {a}.."
        expect = before[row : row + m].double().sum(0)
        assert float((bias_grad[e].double() - expect).abs().max()) <= 2**-7 * max(float(expect.abs().max()), 1.0), f"bias gradient, group {e}"
        row += m


def test_continuous_count_past_2_31_ids():
    n = 2**31 + 1000  # the entry point takes up to 2^32 - 1 ids
    ids = torch.randint(0, 64, (n,), device=DEV, dtype=torch.int32)
    out = continuous_count(x=ids, size=64)
    expect = torch.zeros(64, dtype=torch.int64, device=DEV)
    for a, b in _chunks(n, 2**28):
        expect += torch.bincount(ids[a:b], minlength=64)
    assert torch.equal(out.long(), expect)


def test_router_past_2_32_bytes_of_tokens():
    T, H, E, k = 600000, 4096, 8, 2
    x = torch.randn(T, H, device=DEV, dtype=BF16)
    gate_weight = (torch.randn(E, H, device=DEV) * 0.02).to(BF16)
    logits, weights, selected = C.fused_router(x, gate_weight, k)
    for a, b in _chunks(T, 65536):
        l2, w2, s2 = C.fused_router(x[a:b].contiguous(), gate_weight, k)
        assert torch.equal(l2, logits[a:b]) and torch.equal(w2, weights[a:b]) and torch.equal(s2, selected[a:b]), f"tokens {a}.."
