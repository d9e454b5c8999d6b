"""Pins the CPU oracle (oracle/) without the reference: library routines, closed forms, invariants, brute force and
the reference's own known-answer constructions, chosen so that a dropped term, a wrong index or a transposed operand
fails at least one of them."""

import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import c_oracle, moe_oracle as O
from synthetic_inputs import make_routing


# ---- continuous_count --------------------------------------------------------------------------------------


@pytest.mark.parametrize("impl", [O.continuous_count, c_oracle.continuous_count])
@pytest.mark.parametrize("dtype", [np.int32, np.int64])
def test_count_matches_bincount(impl, dtype):
    # the reference's generator: randint(0, 72), seed 42 (tests/ops/continuous_count_test.py:36-41)
    torch.manual_seed(42)
    for n in [1, 2, 63, 64, 65, 1000, 4097, 100003]:
        x = torch.randint(0, 72, (n,)).numpy().astype(dtype)
        assert np.array_equal(impl(x, 72), np.bincount(x, minlength=72).astype(np.uint32))


@pytest.mark.parametrize("impl", [O.continuous_count, c_oracle.continuous_count])
def test_count_closed_forms(impl):
    E, n = 64, 10_000
    out = impl(np.full(n, 17, np.int32), E)
    expect = np.zeros(E, np.uint32)
    expect[17] = n
    assert np.array_equal(out, expect)
    out = impl((np.arange(n) % E).astype(np.int32), E)
    assert np.array_equal(out, np.array([n // E + (1 if e < n % E else 0) for e in range(E)], np.uint32))
    assert np.array_equal(impl(np.zeros(0, np.int32), E), np.zeros(E, np.uint32))


@pytest.mark.parametrize("impl", [O.continuous_count, c_oracle.continuous_count])
def test_count_brute_force_and_out_of_range(impl):
    rng = np.random.default_rng(0)
    x = rng.integers(-3, 12, size=777).astype(np.int64)
    expect = np.zeros(8, np.uint32)
    for v in x.tolist():
        if 0 <= v < 8:
            expect[v] += 1
    assert np.array_equal(impl(x, 8), expect)
    assert int(impl(x, 8).sum()) == int(((x >= 0) & (x < 8)).sum())


def test_count_size_one_shortcut():
    # size == 1 returns the element count whatever the values are (fma/ops/continuous_count/__init__.py:29-30)
    assert np.array_equal(O.continuous_count(np.array([5, 7, 9], np.int32), 1), np.array([3], np.uint32))


# ---- routing index -------------------------------------------------------------------------------------------


@pytest.mark.parametrize("impl", [O.routing_index, c_oracle.routing_index])
@pytest.mark.parametrize("T,E,k,kind", [(7, 8, 2, "uniform"), (512, 8, 2, "uniform"), (300, 64, 8, "zipf"), (129, 128, 8, "uniform")])
def test_index_matches_stable_sort(impl, T, E, k, kind):
    selected, _ = make_routing(T, E, k, kind, seed=3, empty_tail=4 if kind == "zipf" else 0)
    idx = impl(selected.numpy(), E)
    flat = selected.flatten()
    sorted_ids, sorted_slots = flat.sort(stable=True)
    assert np.array_equal(idx["perm"], sorted_slots.numpy().astype(np.int32))
    assert np.array_equal(idx["eid"], sorted_ids.numpy().astype(np.int32))
    assert np.array_equal(idx["counts"], np.bincount(flat.numpy(), minlength=E).astype(np.uint32))
    assert np.array_equal(idx["offsets"], np.cumsum(idx["counts"]).astype(np.uint32))
    R = T * k
    assert np.array_equal(np.sort(idx["perm"]), np.arange(R, dtype=np.int32))  # a permutation
    assert np.array_equal(idx["inv"][idx["perm"]], np.arange(R, dtype=np.int32))  # its inverse
    assert (np.diff(idx["eid"]) >= 0).all()
    if kind == "zipf":
        assert (idx["counts"][-4:] == 0).all()  # the forced-empty experts really are empty


def test_index_brute_force_tiny():
    ids = np.array([[2, 0], [1, 2], [0, 1], [2, 1]])
    idx = O.routing_index(ids, 3)
    # slots: 0:2 1:0 2:1 3:2 4:0 5:1 6:2 7:1 -> expert 0: [1,4], expert 1: [2,5,7], expert 2: [0,3,6]
    assert idx["perm"].tolist() == [1, 4, 2, 5, 7, 0, 3, 6]
    assert idx["eid"].tolist() == [0, 0, 1, 1, 1, 2, 2, 2]
    assert idx["counts"].tolist() == [2, 3, 3] and idx["offsets"].tolist() == [2, 5, 8]
    assert idx["inv"].tolist() == [5, 0, 2, 6, 1, 3, 7, 4]


# ---- grouped GEMM ---------------------------------------------------------------------------------------------


def _integer_kat(M_list, N, K, tA, tB, seed=42):
    """the reference's known-answer construction (tests/ops/grouped_gemm_test.py:38-92): bf16 operands that are
    integers in [-8, 8], so fp32 accumulation is exact; expected values come from an int64 matmul here."""
    g = torch.Generator().manual_seed(seed)
    As, Bs, Ds = [], [], []
    for M in M_list:
        a = torch.randint(-8, 9, (K, M) if tA else (M, K), generator=g)
        b = torch.randint(-8, 9, (N, K) if tB else (K, N), generator=g)
        As.append(a)
        Bs.append(b)
        Ds.append(((a.T if tA else a) @ (b.T if tB else b)).reshape(-1))
    A = torch.cat([a.reshape(-1) for a in As]).to(torch.bfloat16)
    B = torch.cat([b.reshape(-1) for b in Bs]).to(torch.bfloat16)
    D = torch.cat(Ds)
    return A, B, D


@pytest.mark.parametrize("tA", [False, True])
@pytest.mark.parametrize("tB", [False, True])
def test_grouped_gemm_integer_kat(tA, tB):
    M_list, N, K = [5, 0, 33, 1, 17], 24, 40
    A, B, D = _integer_kat(M_list, N, K, tA, tB)
    out = O.grouped_gemm(A, B, M_list, [N] * 5, [K] * 5, tA, tB)
    expect = D.to(torch.float32).to(torch.bfloat16)  # |D| <= 64*40 fits fp32 exactly, then one RNE to bf16
    assert torch.equal(out, expect)


def test_grouped_gemm_reduces_to_mm_and_bmm():
    torch.manual_seed(0)
    a, b = torch.randn(9, 16), torch.randn(16, 12)
    assert torch.allclose(O.grouped_gemm(a, b, [9], [12], [16]).reshape(9, 12), a @ b, atol=1e-5)
    assert torch.allclose(O.grouped_gemm(a, b.T.contiguous(), [9], [12], [16], False, True).reshape(9, 12), a @ b, atol=1e-5)
    assert torch.allclose(O.grouped_gemm(a.T.contiguous(), b, [9], [12], [16], True, False).reshape(9, 12), a @ b, atol=1e-5)
    a3, b3 = torch.randn(4, 9, 16), torch.randn(4, 16, 12)
    out = O.grouped_gemm(a3, b3, [9] * 4, [12] * 4, [16] * 4, alpha=0.5)
    assert torch.allclose(out.reshape(4, 9, 12), 0.5 * torch.bmm(a3, b3), atol=1e-5)


# ---- SwiGLU ---------------------------------------------------------------------------------------------------


def test_swiglu_closed_forms():
    g = torch.tensor([0.0, 100.0, -100.0, 1.0])
    u = torch.tensor([3.0, 2.0, 2.0, -1.5])
    y = O.swiglu(g, u)
    assert y[0] == 0 and y[1] == 200.0 and abs(float(y[2])) < 1e-30
    assert torch.allclose(y[3], torch.tensor(-1.5 / (1 + np.exp(-1.0)), dtype=torch.float32), atol=1e-7)
    assert torch.equal(O.swiglu(g, u), u * F.silu(g))
    dg, du = O.swiglu_backward(torch.zeros(3), u[:3], torch.ones(3))
    assert torch.allclose(dg, u[:3] / 2) and torch.equal(du, torch.zeros(3))  # gate = 0: dgate = dy*up/2, dup = 0


def test_swiglu_packed_halves_and_derivative():
    torch.manual_seed(1)
    x = torch.randn(5, 8, dtype=torch.float64, requires_grad=True)
    y = O.swiglu_packed(x)
    assert torch.allclose(y, x[:, :4] * F.silu(x[:, 4:]))  # first half up, second half gate
    dy = torch.randn(5, 4, dtype=torch.float64)
    (gx,) = torch.autograd.grad(y, x, dy)
    dg, du = O.swiglu_backward(x[:, 4:].detach().float(), x[:, :4].detach().float(), dy.float())
    assert torch.allclose(gx[:, 4:].float(), dg, atol=1e-5) and torch.allclose(gx[:, :4].float(), du, atol=1e-5)


# ---- routing weights and the layer -----------------------------------------------------------------------------


def test_routing_weights_properties():
    torch.manual_seed(2)
    x, w = torch.randn(33, 16), torch.randn(8, 16)
    logits, weights, selected = O.routing_weights(x, w, 3)
    assert torch.allclose(logits, x @ w.T, atol=1e-6)
    assert torch.allclose(weights.sum(-1), torch.ones(33), atol=1e-6)
    assert torch.equal(selected, logits.topk(3).indices)
    assert torch.allclose(weights, F.softmax(logits.gather(1, selected), -1))
    _, w_all, sel_all = O.routing_weights(x, w, 8)  # k == E: a full softmax, reordered
    assert torch.allclose(torch.zeros(33, 8).scatter(1, sel_all, w_all), F.softmax(logits, -1), atol=1e-6)
    _, w1, s1 = O.routing_weights(x, w, 1)
    assert torch.equal(s1[:, 0], logits.argmax(-1)) and torch.equal(w1, torch.ones(33, 1))


def test_topk_order_against_torch_and_brute_force():
    rng = np.random.default_rng(5)
    # bf16-like logits with many exact ties
    logits = np.round(rng.standard_normal((257, 24)) * 4) / 4
    for k in (1, 2, 5, 24):
        got = O.topk_lowest_index_first(logits, k)
        t = torch.from_numpy(logits)
        # the selected values are what torch.topk selects (the values are unique as a sorted list even with ties)
        assert torch.equal(t.gather(1, torch.from_numpy(got)), t.topk(k, dim=-1).values)
        # and the order is that of a stable descending sort
        assert np.array_equal(got, torch.sort(t, dim=-1, descending=True, stable=True).indices[:, :k].numpy())
    # brute force: repeatedly take the first maximum
    for row in logits[:40]:
        left, expect = list(enumerate(row)), []
        for _ in range(6):
            best = max(v for _, v in left)
            idx = min(i for i, v in left if v == best)
            expect.append(idx)
            left = [(i, v) for i, v in left if i != idx]
        assert list(O.topk_lowest_index_first(row[None], 6)[0]) == expect
    # NaN ranks first (torch.topk's convention), lowest column first among NaNs
    nan_row = np.array([[0.5, np.nan, 3.0, np.nan, 3.0]])
    assert list(O.topk_lowest_index_first(nan_row, 4)[0]) == [1, 3, 2, 4]
    assert list(torch.from_numpy(nan_row).topk(2).indices[0].sort().values) == [1, 3]


def test_router_from_logits_and_its_gradient():
    torch.manual_seed(4)
    x, w = torch.randn(50, 32), torch.randn(12, 32)
    logits, weights, selected = O.routing_weights(x, w, 4)  # continuous random logits: no ties
    w2, s2 = O.router_from_logits(logits, 4)
    assert torch.equal(s2, selected) and torch.equal(w2, weights)

    # gradient: closed form of softmax backward scattered to the kept columns, plus the direct term; the softmax
    # itself runs in fp32 as in the reference (values.float()), hence the 1e-6
    logits64 = logits.double()
    dw, dl = torch.randn(50, 4).double(), torch.randn(50, 12).double()
    got = O.router_logits_grad(logits64, selected, dw, dl)
    s = F.softmax(logits64.gather(1, selected), dim=-1)
    ds = s * (dw - (s * dw).sum(-1, keepdim=True))
    assert torch.allclose(got, dl.clone().scatter_add(1, selected, ds), atol=1e-6, rtol=0)
    assert torch.allclose(O.router_logits_grad(logits64, selected, dw, None), torch.zeros(50, 12).double().scatter_add(1, selected, ds), atol=1e-6, rtol=0)
    assert torch.equal(O.router_logits_grad(logits64, selected, None, dl), dl)
    # shifting all logits of a token leaves the weights unchanged: the rows of the softmax part sum to zero
    assert float(O.router_logits_grad(logits64, selected, dw, None).sum(-1).abs().max()) < 1e-6


def test_fused_residual_add_rmsnorm_definition_and_invariants():
    torch.manual_seed(8)
    x, res, w = torch.randn(19, 37).double(), torch.randn(19, 37).double(), torch.randn(37).double()
    for weight in (None, w):
        for mult in (None, 0.9):
            out, r = O.fused_residual_add_rmsnorm(x, res, weight, 1e-5, mult)
            r_expect = x * (1.0 if mult is None else mult) + res
            assert torch.allclose(r, r_expect, atol=1e-14)
            expect = r_expect / torch.sqrt((r_expect**2).mean(-1, keepdim=True) + 1e-5)
            if weight is not None:
                expect = expect * weight
            assert torch.allclose(out, expect, atol=1e-12)
    # brute force on one row
    out, r = O.fused_residual_add_rmsnorm(x, res, w, 1e-5, 0.9)
    row = [0.9 * float(a) + float(b) for a, b in zip(x[3], res[3])]
    inv = (sum(v * v for v in row) / len(row) + 1e-5) ** -0.5
    assert all(abs(float(out[3, h]) - row[h] * inv * float(w[h])) < 1e-12 for h in range(37))
    # unweighted output has unit root-mean-square (up to eps); scaling the input changes nothing when eps = 0
    out, _ = O.fused_residual_add_rmsnorm(x, res, None, 1e-12)
    assert torch.allclose((out**2).mean(-1), torch.ones(19).double(), atol=1e-9)
    a, _ = O.fused_residual_add_rmsnorm(x, res, w, 0.0)
    b, _ = O.fused_residual_add_rmsnorm(7 * x, 7 * res, w, 0.0)
    assert torch.allclose(a, b, atol=1e-12)
    # eps=None: the dtype's machine epsilon
    c, _ = O.fused_residual_add_rmsnorm(x.float(), res.float(), None, None)
    d, _ = O.fused_residual_add_rmsnorm(x.float(), res.float(), None, torch.finfo(torch.float32).eps)
    assert torch.equal(c, d)
    # gradients of both outputs
    xs, rs, ws = (t[:3, :5].clone().requires_grad_() for t in (x, res, x[:1].expand(3, 37)))
    wv = w[:5].clone().requires_grad_()
    assert torch.autograd.gradcheck(lambda a_, b_, c_: O.fused_residual_add_rmsnorm(a_, b_, c_, 1e-5, 0.9), (xs, rs, wv))


def test_layer_collapses_to_dense_mlp():
    # E = 1, k = 1: softmax of one logit is 1, so the layer is linear -> swiglu -> linear
    torch.manual_seed(3)
    T, H, I = 19, 16, 24
    x, wg = torch.randn(T, H), torch.randn(1, H)
    w1, w2 = torch.randn(1, 2 * I, H) * 0.1, torch.randn(1, H, I) * 0.1
    y, _ = O.moe_layer(x, wg, w1, w2, 1)
    h = x @ w1[0].T
    dense = (h[:, :I] * F.silu(h[:, I:])) @ w2[0].T
    assert torch.allclose(y, dense, atol=1e-5)
    # with biases: a dense MLP with biases
    b1, b2 = torch.randn(1, 2 * I), torch.randn(1, H)
    sel, ones = torch.zeros(T, 1, dtype=torch.long), torch.ones(T, 1)
    yb = O.moe_experts(x, ones, sel, w1, w2, O.swiglu_packed, b1, b2)
    hb = x @ w1[0].T + b1[0]
    assert torch.allclose(yb, (hb[:, :I] * F.silu(hb[:, I:])) @ w2[0].T + b2[0], atol=1e-5)
    # every expert adds its own bias: with zero weights the output is the gate-weighted sum of the chosen biases
    E, k = 5, 2
    sel2, gates = make_routing(T, E, k, "uniform", seed=3)
    bias_out = torch.randn(E, H)
    y0 = O.moe_experts(x, gates, sel2, torch.zeros(E, 2 * I, H), torch.zeros(E, H, I), O.swiglu_packed, None, bias_out)
    assert torch.allclose(y0, (gates.unsqueeze(-1) * bias_out[sel2]).sum(1), atol=1e-6)


def test_layer_against_per_token_loop():
    # brute force: every token visits its k experts one by one
    torch.manual_seed(4)
    T, H, I, E, k = 23, 8, 12, 5, 2
    x = torch.randn(T, H, dtype=torch.float64)
    w1 = torch.randn(E, 2 * I, H, dtype=torch.float64) * 0.3
    w2 = torch.randn(E, H, I, dtype=torch.float64) * 0.3
    selected, weights = make_routing(T, E, k, "uniform", seed=5)
    weights = weights.double()
    y = O.moe_experts(x, weights, selected, w1, w2)
    expect = torch.zeros(T, H, dtype=torch.float64)
    for t in range(T):
        for j in range(k):
            e = int(selected[t, j])
            h = w1[e] @ x[t]
            expect[t] += weights[t, j] * (w2[e] @ (h[:I] * F.silu(h[I:])))
    assert torch.allclose(y, expect, atol=1e-10)


def test_layer_token_permutation_equivariance_and_empty_expert_grads():
    torch.manual_seed(6)
    T, H, I, E, k = 40, 8, 8, 6, 2
    x = torch.randn(T, H, dtype=torch.float64)
    w1 = (torch.randn(E, 2 * I, H, dtype=torch.float64) * 0.3).requires_grad_()
    w2 = (torch.randn(E, H, I, dtype=torch.float64) * 0.3).requires_grad_()
    selected, weights = make_routing(T, E, k, "zipf", seed=7, empty_tail=2)
    weights = weights.double()
    y = O.moe_experts(x, weights, selected, w1, w2)
    p = torch.randperm(T)
    assert torch.allclose(O.moe_experts(x[p], weights[p], selected[p], w1, w2), y[p], atol=1e-12)
    y.sum().backward()
    assert torch.equal(w1.grad[-2:], torch.zeros_like(w1.grad[-2:]))  # experts without tokens: exact zeros
    assert torch.equal(w2.grad[-2:], torch.zeros_like(w2.grad[-2:]))
    assert w1.grad[:4].abs().sum() > 0


def test_layer_gradcheck_fp64():
    torch.manual_seed(8)
    T, H, I, E, k = 6, 4, 4, 3, 2
    selected, weights = make_routing(T, E, k, "uniform", seed=9)
    x = torch.randn(T, H, dtype=torch.float64, requires_grad=True)
    g = weights.double().requires_grad_()
    w1 = (torch.randn(E, 2 * I, H, dtype=torch.float64) * 0.5).requires_grad_()
    w2 = (torch.randn(E, H, I, dtype=torch.float64) * 0.5).requires_grad_()
    assert torch.autograd.gradcheck(lambda a, b, c, d: O.moe_experts(a, b, selected, c, d), (x, g, w1, w2))


def test_golden_fixture_is_what_the_oracle_computes():
    import os

    from tests.golden.make_golden import c1_inputs

    fx = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "c1_moe_fp32.npz"))
    x, wg, w1, w2 = c1_inputs()
    assert abs(float(x.double().sum()) - float(fx["x_sum"])) < 1e-6
    _, weights, selected = O.routing_weights(x, wg, 2)
    assert np.array_equal(selected.numpy(), fx["selected"])
    y = O.moe_experts(x, weights, selected, w1, w2)
    assert np.allclose(y.numpy(), fx["y"], atol=1e-6)
    idx = O.routing_index(selected.numpy(), 8)
    assert np.array_equal(idx["perm"], fx["perm"]) and np.array_equal(idx["counts"], fx["counts"])


GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.mark.parametrize("count,index", [(O.continuous_count, O.routing_index), (c_oracle.continuous_count, c_oracle.routing_index)])
def test_routing_index_fixture(count, index):
    # 4096 skewed ids with three empty experts; the stored answers come from numpy's bincount / cumsum / stable argsort
    fx = np.load(os.path.join(GOLDEN, "routing_index_4096.npz"))
    assert np.array_equal(count(fx["ids"], 64), fx["counts"])
    assert np.array_equal(count(fx["ids"].astype(np.int64), 64), fx["counts"])
    idx = index(fx["ids"], 64)
    for key in ("counts", "offsets", "perm", "eid", "inv"):
        assert np.array_equal(idx[key], fx[key]), key


@pytest.mark.parametrize("layout", ["NT", "NN", "TN", "TT"])
def test_grouped_gemm_known_answer_fixture(layout):
    # the stored products are int64 matrix products of the regenerated integer operands
    from tests.golden.make_golden import kat_problem

    fx = np.load(os.path.join(GOLDEN, "grouped_gemm_kat.npz"))
    M, N, K, tA, tB, As, Bs = kat_problem(layout)
    A = torch.from_numpy(np.concatenate([a.reshape(-1) for a in As])).float()
    B = torch.from_numpy(np.concatenate([b.reshape(-1) for b in Bs])).float()
    got = O.grouped_gemm(A, B, M, N, K, tA, tB)
    assert got.dtype == torch.float32 and np.array_equal(got.numpy().astype(np.int64), fx[layout])
    got16 = O.grouped_gemm(A.bfloat16(), B.bfloat16(), M, N, K, tA, tB)  # operands exact in bf16, one rounding of the result
    assert torch.equal(got16, torch.from_numpy(fx[layout]).float().bfloat16())
