"""CPU oracle of the MoE-layer hot path: TEST INFRASTRUCTURE, not product code.

A restatement, in numpy (integer work) and eager torch (floating point), of what the reference's torch backend
computes for this path. Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may import it;
the product package (cute-kernels_amd/fma) never does.

Every function cites the reference lines it restates (paths relative to the cute-kernels tree). How each one is
pinned (tests/test_oracle.py):
  continuous_count        numpy.bincount, closed forms (constant ids, arange % E, empty), brute-force loop
  routing_index           torch.sort(stable=True), permutation / monotonicity / inverse invariants, brute force
  grouped_gemm            the reference's integer known-answer construction (tests/ops/grouped_gemm_test.py:38-92),
                          E=1 == torch.mm, equal groups == torch.bmm, all four layouts
  swiglu / swiglu_packed  F.silu, closed forms at gate=0, saturation, README derivative vs fp64 autograd
  routing_weights         softmax of top-k logits; k == E reduces to a full softmax
  topk_lowest_index_first torch.topk's values, torch.sort(descending, stable) order, brute force with ties and NaN
  router_from_logits      routing_weights on tie-free logits
  router_logits_grad      closed form s * (dw - <s, dw>) scattered to the kept columns; rows sum to zero
  moe_experts / moe_layer E=1,k=1 collapses to a dense SwiGLU MLP; token-permutation equivariance; zero-token
                          experts get exactly zero weight gradient; fp64 gradcheck on a tiny layer
  fused_residual_add_rmsnorm  the definition written out in fp64 (r / sqrt(mean(r^2) + eps) * w), unit RMS of the
                          unweighted output, invariance to scaling the input (eps = 0), fp64 gradcheck
No function here is "parity unpinned".
"""

from typing import Callable

import numpy as np
import torch
import torch.nn.functional as F


# ---- integer part ------------------------------------------------------------------------------------------


def continuous_count(x: np.ndarray, size: int) -> np.ndarray:
    """out[v] = #{i : x[i] == v} for v in [0, size), uint32; ids outside the range are not counted.

    Restates continuous_count(kernel_backend=torch): `x.bincount(minlength=size).to(uint32)`
    (fma/ops/continuous_count/__init__.py:29-36), including the size == 1 shortcut (:29-30) which returns the
    element count without looking at the values. The docstring there (:15-17) says out-of-range values are ignored.
    """
    x = np.asarray(x)
    if size == 1:
        return np.array([x.size], dtype=np.uint32)
    assert x.ndim == 1 and x.dtype in (np.int32, np.int64)
    out = np.zeros(size, dtype=np.uint32)
    in_range = (x >= 0) & (x < size)
    np.add.at(out, x[in_range], 1)
    return out


def routing_index(selected_experts: np.ndarray, num_experts: int) -> dict[str, np.ndarray]:
    """Expert-major order of the flattened (token, choice) slots.

    Restates `selected_experts.flatten().sort()` + continuous_count + `expert_frequency.cumsum(-1)`
    (fma/modules/moe/__init__.py:214-217,249). The reference's sort is not stable, so the order of slots inside one
    expert is unspecified there; the canonical order here is ascending slot (what a stable sort gives).

    Returns counts uint32[E], offsets uint32[E] (inclusive cumsum), perm int32[R] (sorted_scattered_idxs),
    eid int32[R] (sorted_expert_idxs), inv int32[R] with inv[perm[i]] == i.
    """
    ids = np.asarray(selected_experts).reshape(-1)
    R = ids.size
    counts = continuous_count(ids.astype(np.int64), num_experts) if num_experts > 1 else np.array([R], np.uint32)
    offsets = np.cumsum(counts.astype(np.int64)).astype(np.uint32)
    # counting sort written out: next free position per expert, slots visited in ascending order
    cursor = (offsets.astype(np.int64) - counts.astype(np.int64)).copy()
    perm = np.empty(R, dtype=np.int32)
    inv = np.empty(R, dtype=np.int32)
    # vectorised form of:  for s in range(R): e = ids[s]; perm[cursor[e]] = s; inv[s] = cursor[e]; cursor[e] += 1
    for e in range(num_experts):
        slots = np.nonzero(ids == e)[0]
        pos = cursor[e] + np.arange(slots.size)
        perm[pos] = slots
        inv[slots] = pos
    eid = ids[perm].astype(np.int32)
    return {"counts": counts, "offsets": offsets, "perm": perm, "eid": eid, "inv": inv}


# ---- floating-point part --------------------------------------------------------------------------------------


def grouped_gemm(
    A: torch.Tensor,
    B: torch.Tensor,
    M_array: list[int],
    N_array: list[int],
    K_array: list[int],
    is_A_transposed: bool = False,
    is_B_transposed: bool = False,
    alpha: float = 1.0,
) -> torch.Tensor:
    """Flat packed output of D_e = alpha * op(A_e) @ op(B_e), accumulated in fp32 and rounded to A's dtype.

    Restates the semantics of grouped_gemm (fma/ops/grouped_gemm/__init__.py:11-46): groups packed back to back
    with element offsets sum(M*K), sum(K*N), sum(M*N) (cuda_implementation/kernel.cu:82-90,112-117);
    is_A_transposed=False => A_e stored [M, K], True => [K, M]; is_B_transposed=True => B_e stored [N, K],
    False => [K, N] (kernel.cu:152-154, and the expected values of tests/ops/grouped_gemm_test.py:79-90).
    """
    A, B = A.reshape(-1), B.reshape(-1)
    outs = []
    oa = ob = 0
    for M, N, K in zip(M_array, N_array, K_array):
        a = A[oa : oa + M * K].reshape((K, M) if is_A_transposed else (M, K)).float()
        b = B[ob : ob + K * N].reshape((N, K) if is_B_transposed else (K, N)).float()
        if is_A_transposed:
            a = a.T
        if is_B_transposed:
            b = b.T
        outs.append((alpha * (a @ b)).to(A.dtype).reshape(-1))
        oa += M * K
        ob += K * N
    return torch.cat(outs) if outs else A.new_empty(0)


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """up * silu(gate) in fp32, cast back: the torch branch of swiglu (fma/ops/swiglu/__init__.py:118-126)."""
    dtype = gate.dtype
    wide = torch.float64 if dtype == torch.float64 else torch.float32  # fp64 stays fp64 (used only to pin gradients)
    return (up.to(wide) * F.silu(gate.to(wide))).to(dtype)


def swiglu_packed(x: torch.Tensor) -> torch.Tensor:
    """`up, gate = x.chunk(2, -1)`: first half up, second half gate (fma/ops/swiglu/__init__.py:152-160)."""
    up, gate = x.chunk(2, dim=-1)
    return swiglu(gate, up)


def swiglu_backward(gate: torch.Tensor, up: torch.Tensor, dy: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """(gate_grad, up_grad) from the closed form of fma/ops/swiglu/README.md:12-17:
    dL/du = dy * g * s(g),  dL/dg = dy * u * s(g) * (1 + g - g * s(g))."""
    g, u, d = gate.float(), up.float(), dy.float()
    s = torch.sigmoid(g)
    return (d * u * s * (1 + g - g * s)).to(gate.dtype), (d * g * s).to(up.dtype)


def routing_weights(
    hidden_states: torch.Tensor, gate_weight: torch.Tensor, top_k: int
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(router_logits [T,E], router_weights [T,k], selected_experts [T,k]).

    Restates MoE._compute_routing_weights and _get_topk (fma/modules/moe/__init__.py:191-204,292-298): linear
    without bias, top-k (max when k == 1), softmax over the k kept logits in fp32, cast to the activation dtype.
    """
    router_logits = F.linear(hidden_states, gate_weight)
    if top_k == 1:
        values, selected = router_logits.max(dim=-1, keepdim=True)
    else:
        values, selected = router_logits.topk(top_k, dim=-1)
    weights = F.softmax(values.float(), dim=-1).type_as(hidden_states)
    return router_logits, weights, selected


def topk_lowest_index_first(logits: np.ndarray, top_k: int) -> np.ndarray:
    """int64 [T, k]: columns of the k largest entries of every row, largest first, equal values in ascending column
    order, NaN ranked above every number. torch.topk / torch.max (fma/modules/moe/__init__.py:292-298) fix the
    selected VALUES; among equal values they leave the choice and the order open, and this is the one order the
    fused router kernel is specified to return."""
    a = np.asarray(logits, dtype=np.float64)
    key = np.where(np.isnan(a), np.inf, a)
    # a stable sort of the negated keys keeps equal values in ascending column order
    return np.argsort(-key, axis=-1, kind="stable")[:, :top_k].astype(np.int64)


def router_from_logits(router_logits: torch.Tensor, top_k: int) -> tuple[torch.Tensor, torch.Tensor]:
    """(router_weights [T,k] in the logits' dtype, selected_experts [T,k] int64) from given logits: the part of
    MoE._compute_routing_weights after the gate (fma/modules/moe/__init__.py:196-202) with the tie order above."""
    selected = torch.from_numpy(topk_lowest_index_first(router_logits.detach().float().cpu().numpy(), top_k))
    values = router_logits.detach().cpu().gather(1, selected)
    weights = F.softmax(values.float(), dim=-1).to(router_logits.dtype)
    return weights, selected


def router_logits_grad(
    router_logits: torch.Tensor,
    selected: torch.Tensor,
    weights_grad: torch.Tensor | None,
    logits_output_grad: torch.Tensor | None,
) -> torch.Tensor:
    """Gradient reaching router_logits through autograd of fma/modules/moe/__init__.py:196-202 (gather of the kept
    logits = what topk's backward scatters through, .float(), softmax, cast back) when router_weights receives
    weights_grad and router_logits itself (returned by MoE.forward for auxiliary losses) receives logits_output_grad."""
    logits = router_logits.detach().cpu().clone().requires_grad_()
    values = logits.gather(1, selected.cpu().long())
    weights = F.softmax(values.float(), dim=-1).to(logits.dtype)
    outputs, grads = [], []
    if weights_grad is not None:
        outputs.append(weights)
        grads.append(weights_grad.detach().cpu())
    if logits_output_grad is not None:
        outputs.append(logits * 1)
        grads.append(logits_output_grad.detach().cpu())
    if not outputs:
        return torch.zeros_like(logits)
    torch.autograd.backward(outputs, grads)
    return logits.grad.detach()


def moe_experts(
    hidden_states: torch.Tensor,
    router_weights: torch.Tensor,
    selected_experts: torch.Tensor,
    w_fc: torch.Tensor,
    w_proj: torch.Tensor,
    activation: Callable[[torch.Tensor], torch.Tensor] = swiglu_packed,
    b_fc: torch.Tensor | None = None,
    b_proj: torch.Tensor | None = None,
) -> torch.Tensor:
    """The torch branch of MoE._compute_experts (fma/modules/moe/__init__.py:267-286) with Experts.torch_forward
    (:94-110): sort slots by expert, gather x[slot // k], per-expert F.linear, activation, per-expert F.linear,
    scale by the gathered router weights, index_add back to tokens. Differentiable (autograd gives the oracle's
    gradients). w_fc: [E, 2I or I, H]; w_proj: [E, H, I]; optional biases b_fc: [E, 2I or I], b_proj: [E, H]
    (F.linear(x_e, W[e], bias[e]), :103-105).
    """
    T, H = hidden_states.shape
    E = w_fc.size(0)
    top_k = selected_experts.size(1)
    index = routing_index(selected_experts.detach().cpu().numpy(), E)
    perm = torch.from_numpy(index["perm"].astype(np.int64)).to(hidden_states.device)
    counts = [int(c) for c in index["counts"]]

    fan_in_index = perm // top_k  # :269
    batch_gates = router_weights.flatten()[perm]  # :272-273
    x = hidden_states[fan_in_index]  # :275
    xs = x.split(counts, dim=0)  # :98
    hs = [F.linear(xs[e], w_fc[e], None if b_fc is None else b_fc[e]) for e in range(E)]  # :102-105
    hs = [activation(h) for h in hs]  # :281
    ys = torch.cat([F.linear(hs[e], w_proj[e], None if b_proj is None else b_proj[e]) for e in range(E)], dim=0)  # :282
    ys = ys * batch_gates.unsqueeze(-1)  # :284
    zeros = torch.zeros((T, H), dtype=ys.dtype, device=ys.device)
    return zeros.index_add(0, fan_in_index, ys)  # :285-286


def moe_layer(
    hidden_states: torch.Tensor,
    gate_weight: torch.Tensor,
    w_fc: torch.Tensor,
    w_proj: torch.Tensor,
    top_k: int,
    activation: Callable[[torch.Tensor], torch.Tensor] = swiglu_packed,
) -> tuple[torch.Tensor, torch.Tensor]:
    """MoE.forward (fma/modules/moe/__init__.py:167-189): returns (hidden_states, router_logits)."""
    shape = hidden_states.shape
    x = hidden_states.reshape(-1, shape[-1])
    router_logits, weights, selected = routing_weights(x, gate_weight, top_k)
    y = moe_experts(x, weights, selected, w_fc, w_proj, activation)
    return y.reshape(shape), router_logits


def fused_residual_add_rmsnorm(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor | None, eps: float | None, multiplier: float | None = None
) -> tuple[torch.Tensor, torch.Tensor]:
    """(normalised activations, updated residual stream): the torch branch of fused_residual_add_rmsnorm
    (fma/ops/fused_residual_add_rmsnorm/__init__.py:113-120): optional pre-multiplication of x, residual add,
    F.rms_norm over the last dimension (eps=None means the dtype's machine epsilon, as torch defines it)."""
    if multiplier not in [None, 1]:
        x = x * multiplier
    x = x + residual
    residual = x
    x = F.rms_norm(x, (x.size(-1),), weight=weight, eps=eps)
    return x, residual
