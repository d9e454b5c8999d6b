"""GPU side of the MoE layer: custom ops over libfma_hip.so and the autograd functions built from them.

Stands in for the reference's fma/modules/moe/cuda_implementation/__init__.py (grouped-GEMM experts, group /
ungroup row movement) and for the row kernels of fma/modules/moe/triton_implementation/. Differences by design:
 * no padding: the HIP grouped GEMM masks ragged group edges, so rows are packed back to back (the reference pads
   every group to a multiple of 8 rows for its TMA kernel, cuda_implementation/__init__.py:83-104);
 * the routed order is built by a stable counting sort (counts -> offsets -> placement) that also yields the
   inverse permutation, which makes the combine and every backward gather atomic-free and deterministic;
 * index tensors are int32.
"""

import torch
from torch.library import custom_op

from ... import _lib
from ...constants import LIBRARY_NAME
from ...ops import grouped_gemm
from ...utils import ensure_contiguous


# ---- custom ops ---------------------------------------------------------------------------------


@custom_op(f"{LIBRARY_NAME}::moe_build_index_cuda", mutates_args={"counts", "offsets", "perm", "eid", "inv"})
def moe_build_index_cuda(
    ids: torch.Tensor,
    counts: torch.Tensor,
    offsets: torch.Tensor,
    perm: torch.Tensor,
    eid: torch.Tensor,
    inv: torch.Tensor,
) -> None:
    _lib.require_gpu(ids, counts, offsets, perm, eid, inv)
    assert ids.dtype in (torch.int32, torch.int64) and ids.is_contiguous()
    assert counts.dtype == torch.uint32 and offsets.dtype == torch.uint32
    assert perm.dtype == eid.dtype == inv.dtype == torch.int32
    R, E = ids.numel(), counts.numel()
    assert perm.numel() == eid.numel() == inv.numel() == R and offsets.numel() == E
    lib = _lib.load()
    with torch.cuda.device(ids.device):
        # per-chunk histograms; scratch owned by this call (the op body is opaque to tracing, so the size query
        # and the allocation may live here)
        nbytes = max(lib.fma_moe_build_index_workspace_bytes(R, E), 4)
        workspace = torch.empty(nbytes, dtype=torch.uint8, device=ids.device)
        rc = lib.fma_moe_build_index(
            ids.data_ptr(), ids.element_size(), R, E, counts.data_ptr(), offsets.data_ptr(), perm.data_ptr(),
            eid.data_ptr(), inv.data_ptr(), workspace.data_ptr(), nbytes, _lib.current_stream(ids.device),
        )
    _lib.check(rc, "moe_build_index_cuda")


@custom_op(
    f"{LIBRARY_NAME}::moe_build_index_from_hist_cuda",
    mutates_args={"token_block_hist", "counts", "offsets", "perm", "eid", "inv"},
)
def moe_build_index_from_hist_cuda(
    ids: torch.Tensor,
    top_k: int,
    token_block_hist: torch.Tensor,
    counts: torch.Tensor,
    offsets: torch.Tensor,
    perm: torch.Tensor,
    eid: torch.Tensor,
    inv: torch.Tensor,
) -> None:
    """moe_build_index_cuda for choices the fused router has already counted per block of 16 tokens: scan and
    placement only. The histogram serves as scratch memory and is overwritten."""
    _lib.require_gpu(ids, token_block_hist, counts, offsets, perm, eid, inv)
    assert ids.dtype == torch.int32 and ids.is_contiguous()
    assert counts.dtype == torch.uint32 and offsets.dtype == torch.uint32
    assert perm.dtype == eid.dtype == inv.dtype == torch.int32
    R, E = ids.numel(), counts.numel()
    assert perm.numel() == eid.numel() == inv.numel() == R and offsets.numel() == E and R % top_k == 0
    assert token_block_hist.dtype == torch.uint32 and token_block_hist.is_contiguous()
    assert token_block_hist.shape == ((R // top_k + 15) // 16, E)
    with torch.cuda.device(ids.device):
        rc = _lib.load().fma_moe_build_index_from_hist(
            ids.data_ptr(), R, E, top_k, _lib.ptr(token_block_hist), counts.data_ptr(), offsets.data_ptr(),
            perm.data_ptr(), eid.data_ptr(), inv.data_ptr(), _lib.current_stream(ids.device),
        )
    _lib.check(rc, "moe_build_index_from_hist_cuda")


@custom_op(f"{LIBRARY_NAME}::gather_rows_cuda", mutates_args={"output"})
def gather_rows_cuda(x: torch.Tensor, idx: torch.Tensor, divisor: int, output: torch.Tensor) -> None:
    _lib.require_gpu(x, idx, output)
    assert x.dim() == 2 and output.dim() == 2 and x.size(1) == output.size(1) and x.dtype == output.dtype
    assert idx.dtype == torch.int32 and idx.numel() == output.size(0)  # x may have more rows than are gathered
    assert x.is_contiguous() and output.is_contiguous() and idx.is_contiguous()
    with torch.cuda.device(x.device):
        rc = _lib.load().fma_gather_rows(
            x.data_ptr(), idx.data_ptr(), output.size(0), x.size(1), divisor, output.data_ptr(),
            _lib.dtype_code(x.dtype), _lib.current_stream(x.device),
        )
    _lib.check(rc, "gather_rows_cuda")


@custom_op(f"{LIBRARY_NAME}::dispatch_rows_cuda", mutates_args={"output"})
def dispatch_rows_cuda(x: torch.Tensor, inv: torch.Tensor, top_k: int, output: torch.Tensor) -> None:
    _lib.require_gpu(x, inv, output)
    T, H = x.shape
    # at least one destination row per (token, choice); more when the destination is a padded layout
    assert output.dim() == 2 and output.size(0) >= T * top_k and output.size(1) == H and x.dtype == output.dtype
    assert inv.dtype == torch.int32 and inv.numel() == T * top_k
    assert x.is_contiguous() and output.is_contiguous() and inv.is_contiguous()
    with torch.cuda.device(x.device):
        rc = _lib.load().fma_dispatch_rows(
            x.data_ptr(), inv.data_ptr(), T, top_k, H, output.data_ptr(), _lib.dtype_code(x.dtype),
            _lib.current_stream(x.device),
        )
    _lib.check(rc, "dispatch_rows_cuda")


@custom_op(f"{LIBRARY_NAME}::combine_cuda", mutates_args={"output"})
def combine_cuda(
    o: torch.Tensor, inv: torch.Tensor, gates: torch.Tensor | None, top_k: int, output: torch.Tensor
) -> None:
    _lib.require_gpu(o, inv, gates, output)
    T, H = output.shape
    assert o.dim() == 2 and o.size(1) == H and o.dtype == output.dtype
    assert inv.dtype == torch.int32 and inv.numel() == T * top_k
    assert gates is None or (gates.dtype == o.dtype and gates.numel() == T * top_k and gates.is_contiguous())
    assert o.is_contiguous() and output.is_contiguous() and inv.is_contiguous()
    with torch.cuda.device(o.device):
        rc = _lib.load().fma_combine(
            o.data_ptr(), inv.data_ptr(), _lib.ptr(gates), T, top_k, H, output.data_ptr(), _lib.dtype_code(o.dtype),
            _lib.current_stream(o.device),
        )
    _lib.check(rc, "combine_cuda")


@custom_op(f"{LIBRARY_NAME}::combine_backward_cuda", mutates_args={"o_grad", "gates_grad"})
def combine_backward_cuda(
    output_grad: torch.Tensor,
    o: torch.Tensor,
    inv: torch.Tensor,
    gates: torch.Tensor | None,
    top_k: int,
    o_grad: torch.Tensor,
    gates_grad: torch.Tensor | None,
) -> None:
    _lib.require_gpu(output_grad, o, inv, gates, o_grad, gates_grad)
    T, H = output_grad.shape
    assert o.shape == o_grad.shape and o.size(1) == H
    assert output_grad.dtype == o.dtype == o_grad.dtype
    assert inv.dtype == torch.int32 and inv.numel() == T * top_k
    for t in (output_grad, o, o_grad, inv, gates, gates_grad):
        assert t is None or t.is_contiguous()
    assert gates is None or gates.dtype == o.dtype
    assert gates_grad is None or (gates_grad.dtype == o.dtype and gates_grad.numel() == T * top_k)
    with torch.cuda.device(o.device):
        rc = _lib.load().fma_combine_bwd(
            output_grad.data_ptr(), o.data_ptr(), inv.data_ptr(), _lib.ptr(gates), T, top_k, H, o_grad.data_ptr(),
            _lib.ptr(gates_grad), _lib.dtype_code(o.dtype), _lib.current_stream(o.device),
        )
    _lib.check(rc, "combine_backward_cuda")


@custom_op(f"{LIBRARY_NAME}::grouped_gemm_ragged_cuda", mutates_args={"output"})
def grouped_gemm_ragged_cuda(
    A: torch.Tensor, B: torch.Tensor, output: torch.Tensor, sizes: torch.Tensor, vary_k: bool, M: int, N: int, K: int,
    is_A_transposed: bool, is_B_transposed: bool, bias: torch.Tensor | None = None,
) -> None:  # fmt: skip
    """grouped_gemm for groups that differ in one dimension: `sizes` holds the rows of the groups (M is ignored) or, with
    vary_k, their reduction lengths (K is ignored); the other two dimensions are plain integers (fma_grouped_gemm_ragged).
    `bias` [E, N] is added to the rows of every group in the epilogue (forward form only)."""
    _lib.require_gpu(A, B, output, sizes, bias)
    assert A.dtype == B.dtype == output.dtype and A.dtype in (torch.bfloat16, torch.float16)
    assert sizes.dtype == torch.uint32 and sizes.is_contiguous()
    assert A.is_contiguous() and B.is_contiguous() and output.is_contiguous()
    assert bias is None or (bias.shape == (sizes.numel(), N) and bias.dtype == A.dtype and bias.is_contiguous())
    if output.numel() == 0:
        return
    # an operand without elements is never read, but the entry point rejects NULL: any valid device address stands in
    a_ptr = A.data_ptr() if A.numel() else output.data_ptr()
    b_ptr = B.data_ptr() if B.numel() else output.data_ptr()
    with torch.cuda.device(A.device):
        rc = _lib.load().fma_grouped_gemm_ragged(
            a_ptr, b_ptr, output.data_ptr(), sizes.data_ptr(), _lib.ptr(bias), sizes.numel(),
            _lib.FMA_VARY_K if vary_k else _lib.FMA_VARY_M, M, N, K, int(is_A_transposed), int(is_B_transposed), 1.0,
            _lib.dtype_code(A.dtype), _lib.current_stream(A.device),
        )
    _lib.check(rc, "grouped_gemm_ragged_cuda")


def _expert_gemm(
    A: torch.Tensor, B: torch.Tensor, M_array: torch.Tensor, N_array: torch.Tensor, K_array: torch.Tensor,
    output_shape: tuple[int, ...], vary: str, M: int, N: int, K: int, is_A_transposed: bool, is_B_transposed: bool,
    bias: torch.Tensor | None = None,
) -> torch.Tensor:  # fmt: skip
    """One grouped GEMM of the expert path. `vary` names the array that holds the per-expert sizes ("M" or "K" of this
    product); the other two dimensions are the module's constants M, N, K. 16-bit operands go through the entry point
    that takes them by value (the only one with a bias term), fp32 through `grouped_gemm` with the three arrays."""
    if A.dtype in (torch.bfloat16, torch.float16):
        output = A.new_empty(tuple(output_shape))
        sizes = M_array if vary == "M" else K_array
        grouped_gemm_ragged_cuda(A, B, output, sizes, vary == "K", M, N, K, is_A_transposed, is_B_transposed, bias)
        return output
    assert bias is None
    return grouped_gemm(
        A=A, B=B, C=None, M_array=M_array, N_array=N_array, K_array=K_array, output_shape=output_shape,
        is_A_transposed=is_A_transposed, is_B_transposed=is_B_transposed,
    )


@custom_op(f"{LIBRARY_NAME}::grouped_gemm_swiglu_cuda", mutates_args={"h", "act"})
def grouped_gemm_swiglu_cuda(
    x: torch.Tensor, weight: torch.Tensor, M_array: torch.Tensor, h: torch.Tensor | None, act: torch.Tensor,
    bias: torch.Tensor | None = None,
) -> None:  # fmt: skip
    _lib.require_gpu(x, weight, M_array, h, act, bias)
    E, N, K = weight.shape
    assert N % 2 == 0
    inter = N // 2
    R = x.size(0)
    assert x.shape == (R, K) and act.shape == (R, inter) and (h is None or h.shape == (R, N))
    assert x.dtype == weight.dtype == act.dtype and (h is None or h.dtype == x.dtype)
    assert M_array.dtype == torch.uint32 and M_array.numel() == E
    assert bias is None or (bias.shape == (E, N) and bias.dtype == x.dtype)
    for t in (x, weight, M_array, h, act, bias):
        assert t is None or t.is_contiguous()
    if act.numel() == 0:
        return  # no rows routed anywhere (or no output columns): nothing to compute, and empty tensors have no address
    with torch.cuda.device(x.device):
        rc = _lib.load().fma_grouped_gemm_swiglu(
            x.data_ptr(), weight.data_ptr(), _lib.ptr(bias), _lib.ptr(h), act.data_ptr(), M_array.data_ptr(), E, inter, K,
            _lib.dtype_code(x.dtype), _lib.current_stream(x.device),
        )
    _lib.check(rc, "grouped_gemm_swiglu_cuda")


@custom_op(f"{LIBRARY_NAME}::grouped_gemm_swiglu_bwd_cuda", mutates_args={"h_grad"})
def grouped_gemm_swiglu_bwd_cuda(
    output_grad: torch.Tensor, weight: torch.Tensor, h: torch.Tensor, M_array: torch.Tensor, h_grad: torch.Tensor
) -> None:
    """h_grad = backward of swiglu_packed at h applied to (output_grad_e @ W_e), W_e the second projection's [out, in]
    weight: the input gradient of that projection with the activation's backward in its epilogue
    (fma_grouped_gemm_swiglu_bwd)."""
    _lib.require_gpu(output_grad, weight, h, M_array, h_grad)
    E, K, inter = weight.shape
    R = output_grad.size(0)
    assert output_grad.shape == (R, K) and h.shape == (R, 2 * inter) and h_grad.shape == h.shape
    assert output_grad.dtype == weight.dtype == h.dtype == h_grad.dtype and h.dtype in (torch.bfloat16, torch.float16)
    assert M_array.dtype == torch.uint32 and M_array.numel() == E
    for t in (output_grad, weight, h, M_array, h_grad):
        assert t.is_contiguous()
    if R == 0 or inter == 0:
        return
    with torch.cuda.device(h.device):
        rc = _lib.load().fma_grouped_gemm_swiglu_bwd(
            output_grad.data_ptr(), weight.data_ptr(), h.data_ptr(), h_grad.data_ptr(), M_array.data_ptr(), E, inter, K,
            _lib.dtype_code(h.dtype), _lib.current_stream(h.device),
        )
    _lib.check(rc, "grouped_gemm_swiglu_bwd_cuda")


@custom_op(f"{LIBRARY_NAME}::grouped_gemm_gathered_cuda", mutates_args={"out", "act"})
def grouped_gemm_gathered_cuda(
    x: torch.Tensor,
    row_index: torch.Tensor,
    divisor: int,
    weight: torch.Tensor,
    bias: torch.Tensor | None,
    M_array: torch.Tensor,
    out: torch.Tensor | None,
    act: torch.Tensor | None,
) -> None:
    """The forward product of an expert projection on the rows x[row_index[i] // divisor] (i over the packed rows of all
    experts), gathered inside the operand load. act None: out [R, N] = rows @ W^T (+ bias). Otherwise N = 2 I, act [R, I]
    is swiglu_packed of the pre-activation, which is also written to out unless that is None (fma_grouped_gemm_gathered).
    """
    _lib.require_gpu(x, row_index, weight, bias, M_array, out, act)
    E, N, K = weight.shape
    R = row_index.numel()
    assert x.dim() == 2 and x.size(1) == K and x.dtype == weight.dtype and x.dtype in (torch.bfloat16, torch.float16)
    assert row_index.dtype == torch.int32 and M_array.dtype == torch.uint32 and M_array.numel() == E
    assert out is None or (out.shape == (R, N) and out.dtype == x.dtype)
    assert act is None or (N % 2 == 0 and act.shape == (R, N // 2) and act.dtype == x.dtype)
    assert out is not None or act is not None
    assert bias is None or (bias.shape == (E, N) and bias.dtype == x.dtype)
    for t in (x, row_index, weight, bias, M_array, out, act):
        assert t is None or t.is_contiguous()
    if R == 0 or N == 0:
        return
    with torch.cuda.device(x.device):
        rc = _lib.load().fma_grouped_gemm_gathered(
            x.data_ptr(), x.size(0), row_index.data_ptr(), divisor, weight.data_ptr(), _lib.ptr(bias), _lib.ptr(out),
            _lib.ptr(act), M_array.data_ptr(), E, N, K, int(act is not None), _lib.dtype_code(x.dtype),
            _lib.current_stream(x.device),
        )
    _lib.check(rc, "grouped_gemm_gathered_cuda")


@custom_op(f"{LIBRARY_NAME}::grouped_gemm_gathered_wgrad_cuda", mutates_args={"weight_grad"})
def grouped_gemm_gathered_wgrad_cuda(
    output_grad: torch.Tensor,
    x: torch.Tensor,
    row_index: torch.Tensor,
    divisor: int,
    K_array: torch.Tensor,
    weight_grad: torch.Tensor,
) -> None:
    """The weight gradient of an expert projection on the rows x[row_index[i] // divisor] (i over the packed rows of all
    experts, K_array[e] of them for expert e), gathered inside the operand load: weight_grad[e] [N, K] = output_grad_e^T @
    those rows (fma_grouped_gemm_gathered_wgrad)."""
    _lib.require_gpu(output_grad, x, row_index, K_array, weight_grad)
    E, N, K = weight_grad.shape
    R = row_index.numel()
    assert x.dim() == 2 and x.size(1) == K and output_grad.shape == (R, N)
    assert x.dtype == output_grad.dtype == weight_grad.dtype and x.dtype in (torch.bfloat16, torch.float16)
    assert row_index.dtype == torch.int32 and K_array.dtype == torch.uint32 and K_array.numel() == E
    for t in (output_grad, x, row_index, K_array, weight_grad):
        assert t.is_contiguous()
    if weight_grad.numel() == 0:
        return
    if R == 0:
        weight_grad.zero_()
        return
    with torch.cuda.device(x.device):
        rc = _lib.load().fma_grouped_gemm_gathered_wgrad(
            output_grad.data_ptr(), x.data_ptr(), x.size(0), row_index.data_ptr(), divisor, weight_grad.data_ptr(),
            K_array.data_ptr(), E, N, K, 1.0, _lib.dtype_code(x.dtype), _lib.current_stream(x.device),
        )
    _lib.check(rc, "grouped_gemm_gathered_wgrad_cuda")


@custom_op(f"{LIBRARY_NAME}::expert_bias_add_cuda", mutates_args={"y"})
def expert_bias_add_cuda(y: torch.Tensor, bias: torch.Tensor, M_array: torch.Tensor) -> None:
    _lib.require_gpu(y, bias, M_array)
    E, N = bias.shape
    assert y.dim() == 2 and y.size(1) == N and y.dtype == bias.dtype
    assert M_array.dtype == torch.uint32 and M_array.numel() == E
    assert y.is_contiguous() and bias.is_contiguous() and M_array.is_contiguous()
    with torch.cuda.device(y.device):
        rc = _lib.load().fma_expert_bias_add(
            y.data_ptr(), bias.data_ptr(), M_array.data_ptr(), E, y.size(0), N, _lib.dtype_code(y.dtype),
            _lib.current_stream(y.device),
        )
    _lib.check(rc, "expert_bias_add_cuda")


@custom_op(f"{LIBRARY_NAME}::expert_bias_grad_cuda", mutates_args={"bias_grad"})
def expert_bias_grad_cuda(output_grad: torch.Tensor, M_array: torch.Tensor, bias_grad: torch.Tensor) -> None:
    _lib.require_gpu(output_grad, M_array, bias_grad)
    E, N = bias_grad.shape
    assert output_grad.dim() == 2 and output_grad.size(1) == N and output_grad.dtype == bias_grad.dtype
    assert M_array.dtype == torch.uint32 and M_array.numel() == E
    assert output_grad.is_contiguous() and bias_grad.is_contiguous() and M_array.is_contiguous()
    lib = _lib.load()
    code = _lib.dtype_code(output_grad.dtype)
    with torch.cuda.device(output_grad.device):
        nbytes = max(lib.fma_expert_bias_grad_workspace_bytes(E, output_grad.size(0), N), 4)
        workspace = torch.empty(nbytes, dtype=torch.uint8, device=output_grad.device)  # per-slice partial sums
        rc = lib.fma_expert_bias_grad(
            output_grad.data_ptr(), M_array.data_ptr(), E, output_grad.size(0), N, bias_grad.data_ptr(),
            workspace.data_ptr(), nbytes, code, _lib.current_stream(output_grad.device),
        )
    _lib.check(rc, "expert_bias_grad_cuda")


@custom_op(
    f"{LIBRARY_NAME}::router_topk_cuda", mutates_args={"logits", "weights", "selected", "counts", "token_block_hist"}
)
def router_topk_cuda(
    x: torch.Tensor,
    gate_weight: torch.Tensor,
    top_k: int,
    logits: torch.Tensor,
    weights: torch.Tensor,
    selected: torch.Tensor,
    counts: torch.Tensor | None,
    token_block_hist: torch.Tensor | None,
) -> None:
    _lib.require_gpu(x, gate_weight, logits, weights, selected, counts, token_block_hist)
    T, H = x.shape
    E = gate_weight.size(0)
    assert gate_weight.shape == (E, H) and logits.shape == (T, E)
    assert weights.shape == (T, top_k) and selected.shape == (T, top_k)
    assert x.dtype == gate_weight.dtype == logits.dtype == weights.dtype and selected.dtype == torch.int32
    assert counts is None or (counts.dtype == torch.uint32 and counts.numel() == E)
    assert token_block_hist is None or (
        token_block_hist.dtype == torch.uint32 and token_block_hist.shape == ((T + 15) // 16, E)
    )
    for t in (x, gate_weight, logits, weights, selected, counts, token_block_hist):
        assert t is None or t.is_contiguous()
    with torch.cuda.device(x.device):
        rc = _lib.load().fma_router_topk(
            x.data_ptr(), gate_weight.data_ptr(), T, H, E, top_k, logits.data_ptr(), weights.data_ptr(),
            selected.data_ptr(), _lib.ptr(counts), _lib.ptr(token_block_hist), _lib.dtype_code(x.dtype),
            _lib.current_stream(x.device),
        )
    _lib.check(rc, "router_topk_cuda")


@custom_op(f"{LIBRARY_NAME}::router_topk_backward_cuda", mutates_args={"logits_grad"})
def router_topk_backward_cuda(
    logits: torch.Tensor,
    selected: torch.Tensor,
    weights_grad: torch.Tensor | None,
    logits_output_grad: torch.Tensor | None,
    logits_grad: torch.Tensor,
) -> None:
    _lib.require_gpu(logits, selected, weights_grad, logits_output_grad, logits_grad)
    T, E = logits.shape
    top_k = selected.size(1)
    assert selected.shape == (T, top_k) and selected.dtype == torch.int32 and logits_grad.shape == (T, E)
    assert logits_grad.dtype == logits.dtype
    assert weights_grad is None or (weights_grad.shape == (T, top_k) and weights_grad.dtype == logits.dtype)
    assert logits_output_grad is None or (logits_output_grad.shape == (T, E) and logits_output_grad.dtype == logits.dtype)
    for t in (logits, selected, weights_grad, logits_output_grad, logits_grad):
        assert t is None or t.is_contiguous()
    with torch.cuda.device(logits.device):
        rc = _lib.load().fma_router_topk_bwd(
            logits.data_ptr(), selected.data_ptr(), _lib.ptr(weights_grad), _lib.ptr(logits_output_grad), T, E, top_k,
            logits_grad.data_ptr(), _lib.dtype_code(logits.dtype), _lib.current_stream(logits.device),
        )
    _lib.check(rc, "router_topk_backward_cuda")


# ---- index construction -----------------------------------------------------------------------------


@torch.no_grad()
def build_routing_index(
    selected_experts: torch.Tensor, num_experts: int, token_block_histogram: torch.Tensor | None = None
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Stable counting sort of the flattened (token, choice) slots by expert.

    token_block_histogram: what the fused router counted while choosing (per block of 16 tokens); with it the sort is a
    scan and a placement pass, without it the choices are counted first. It is overwritten.

    Returns (expert_frequency uint32[E], expert_offsets uint32[E] (inclusive), sorted_scattered_idxs int32[R],
    sorted_expert_idxs int32[R], inverse int32[R]); the first four are what the reference obtains from
    `selected_experts.flatten().sort()`, continuous_count and cumsum (fma/modules/moe/__init__.py:214-217,249), with
    the order inside one expert fixed to ascending slot.
    """
    ids = selected_experts.reshape(-1).contiguous()
    device = ids.device
    R = ids.numel()
    counts = torch.empty(num_experts, dtype=torch.uint32, device=device)
    offsets = torch.empty(num_experts, dtype=torch.uint32, device=device)
    perm = torch.empty(R, dtype=torch.int32, device=device)
    eid = torch.empty(R, dtype=torch.int32, device=device)
    inv = torch.empty(R, dtype=torch.int32, device=device)
    if token_block_histogram is not None and ids.dtype == torch.int32 and selected_experts.dim() == 2:
        moe_build_index_from_hist_cuda(
            ids, selected_experts.size(1), token_block_histogram, counts, offsets, perm, eid, inv
        )
    else:
        moe_build_index_cuda(ids, counts, offsets, perm, eid, inv)
    return counts, offsets, perm, eid, inv


# ---- autograd functions -----------------------------------------------------------------------------


class _FusedRouter(torch.autograd.Function):
    """(router_logits, router_weights, selected_experts) of MoE._compute_routing_weights
    (fma/modules/moe/__init__.py:191-204) from one kernel. The backward forms the logits' gradient (softmax and top-k
    backward plus whatever arrives for the logits themselves) in one kernel; the two products with it are GEMMs with
    one tiny dimension (E) and go to the BLAS library like the backward of the reference's nn.Linear gate."""

    @staticmethod
    @ensure_contiguous
    def forward(ctx, x: torch.Tensor, gate_weight: torch.Tensor, top_k: int):
        T, E = x.size(0), gate_weight.size(0)
        logits = torch.empty(T, E, device=x.device, dtype=x.dtype)
        weights = torch.empty(T, top_k, device=x.device, dtype=x.dtype)
        selected = torch.empty(T, top_k, device=x.device, dtype=torch.int32)
        # the choices counted per block of 16 tokens, for the index build that follows
        token_block_hist = torch.empty((T + 15) // 16, E, device=x.device, dtype=torch.uint32)
        router_topk_cuda(x, gate_weight, top_k, logits, weights, selected, None, token_block_hist)
        ctx.save_for_backward(x, gate_weight, logits, selected)
        ctx.mark_non_differentiable(selected, token_block_hist)
        ctx.set_materialize_grads(False)
        return logits, weights, selected, token_block_hist

    @staticmethod
    @ensure_contiguous
    def backward(ctx, logits_output_grad, weights_grad, _, __):
        x, gate_weight, logits, selected = ctx.saved_tensors
        if logits_output_grad is None and weights_grad is None:
            return None, None, None
        logits_grad = torch.empty_like(logits)
        router_topk_backward_cuda(logits, selected, weights_grad, logits_output_grad, logits_grad)
        x_grad = logits_grad @ gate_weight if ctx.needs_input_grad[0] else None
        gate_weight_grad = logits_grad.t() @ x if ctx.needs_input_grad[1] else None
        return x_grad, gate_weight_grad, None


def fused_router(x: torch.Tensor, gate_weight: torch.Tensor, top_k: int):
    """(router_logits, router_weights, selected_experts)"""
    return _FusedRouter.apply(x, gate_weight, top_k)[:3]


def fused_router_with_histogram(x: torch.Tensor, gate_weight: torch.Tensor, top_k: int):
    """fused_router plus the uint32 [ceil(T / 16), E] histogram of the choices per block of 16 tokens, which
    build_routing_index takes (and overwrites)"""
    return _FusedRouter.apply(x, gate_weight, top_k)


class _GatherRows(torch.autograd.Function):
    """xg[i] = x[perm[i] // top_k]; backward sums the top_k grouped rows of every token through `inv`."""

    @staticmethod
    @ensure_contiguous
    def forward(ctx, x: torch.Tensor, perm: torch.Tensor, inv: torch.Tensor, top_k: int) -> torch.Tensor:
        assert x.dim() == 2
        output = torch.empty(perm.numel(), x.size(1), device=x.device, dtype=x.dtype)
        # token-side form of output[i] = x[perm[i] // top_k]: every row of x is read once
        dispatch_rows_cuda(x, inv, top_k, output)
        ctx.save_for_backward(inv)
        ctx.top_k = top_k
        ctx.T = x.size(0)
        return output

    @staticmethod
    @ensure_contiguous
    def backward(ctx, output_grad: torch.Tensor) -> tuple[torch.Tensor | None]:
        (inv,) = ctx.saved_tensors
        x_grad = torch.empty(ctx.T, output_grad.size(1), device=output_grad.device, dtype=output_grad.dtype)
        combine_cuda(output_grad, inv, None, ctx.top_k, x_grad)
        return x_grad, None, None, None


class _Combine(torch.autograd.Function):
    """y[t] = sum_j gates[t, j] * o[inv[t*k + j]]."""

    @staticmethod
    @ensure_contiguous
    def forward(ctx, o: torch.Tensor, gates: torch.Tensor, inv: torch.Tensor) -> torch.Tensor:
        T, top_k = gates.shape
        output = torch.empty(T, o.size(1), device=o.device, dtype=o.dtype)
        combine_cuda(o, inv, gates, top_k, output)
        ctx.save_for_backward(o, gates, inv)
        return output

    @staticmethod
    @ensure_contiguous
    def backward(ctx, output_grad: torch.Tensor) -> tuple[torch.Tensor | None]:
        o, gates, inv = ctx.saved_tensors
        o_grad = torch.empty_like(o)
        gates_grad = torch.empty_like(gates) if ctx.needs_input_grad[1] else None
        combine_backward_cuda(output_grad, o, inv, gates, gates.size(1), o_grad, gates_grad)
        return o_grad, gates_grad, None


class _GroupedGemmExperts(torch.autograd.Function):
    """y_e = x_e @ W_e^T (+ bias_e, 16-bit types: added in the GEMM's epilogue) per expert; the three GEMMs of the
    reference's _GroupedGemmExperts (fma/modules/moe/cuda_implementation/__init__.py:15-80)."""

    @staticmethod
    @ensure_contiguous
    def forward(
        ctx, x: torch.Tensor, weight: torch.Tensor, M_array: torch.Tensor, N_array: torch.Tensor, K_array: torch.Tensor,
        bias: torch.Tensor | None = None,
    ) -> torch.Tensor:  # fmt: skip
        # x -> sum(M) x K, weight -> E x N x K
        _, N, K = weight.size()

        assert N % 8 == 0
        assert K % 8 == 0

        output = _expert_gemm(
            x, weight, M_array, N_array, K_array, (x.size(0), N), "M", 0, N, K, is_A_transposed=False, is_B_transposed=True,
            bias=bias,
        )

        ctx.save_for_backward(x, weight, M_array, K_array, N_array)

        return output

    @staticmethod
    @ensure_contiguous
    def backward(ctx, output_grad: torch.Tensor) -> tuple[torch.Tensor | None]:
        x, weight, M_array, K_array, N_array = ctx.saved_tensors
        _, N, K = weight.size()
        x_grad = weight_grad = bias_grad = None

        if ctx.needs_input_grad[0]:
            # dx_e = dy_e @ W_e : A = dy [sum(M), N], B = W_e stored [N, K] as a [K_gemm = N, N_gemm = K] matrix
            x_grad = _expert_gemm(
                output_grad, weight, M_array, K_array, N_array, x.size(), "M", 0, K, N,
                is_A_transposed=False, is_B_transposed=False,
            )

        if ctx.needs_input_grad[1]:
            # dW_e = dy_e^T @ x_e : both operands are stored with the reduction dim (the M_e rows) as row index
            weight_grad = _expert_gemm(
                output_grad, x, N_array, K_array, M_array, weight.size(), "K", N, K, 0,
                is_A_transposed=True, is_B_transposed=False,
            )

        if len(ctx.needs_input_grad) > 5 and ctx.needs_input_grad[5]:
            bias_grad = torch.empty(weight.size(0), N, device=output_grad.device, dtype=output_grad.dtype)
            expert_bias_grad_cuda(output_grad, M_array, bias_grad)

        return (x_grad, weight_grad, None, None, None, bias_grad)[: len(ctx.needs_input_grad)]


class _ExpertBias(torch.autograd.Function):
    """y_e += bias[e] on the packed rows of every expert, in place on the grouped GEMM's fresh output (which no other
    node needs: the GEMM's backward reads its inputs, not its output); backward sums the rows of every expert."""

    @staticmethod
    def forward(ctx, y: torch.Tensor, bias: torch.Tensor, M_array: torch.Tensor) -> torch.Tensor:
        assert y.is_contiguous()
        expert_bias_add_cuda(y, bias.contiguous(), M_array)
        ctx.mark_dirty(y)
        ctx.save_for_backward(M_array)
        ctx.bias_shape = bias.shape
        return y

    @staticmethod
    @ensure_contiguous
    def backward(ctx, output_grad: torch.Tensor) -> tuple[torch.Tensor | None]:
        (M_array,) = ctx.saved_tensors
        bias_grad = None
        if ctx.needs_input_grad[1]:
            bias_grad = torch.empty(ctx.bias_shape, device=output_grad.device, dtype=output_grad.dtype)
            expert_bias_grad_cuda(output_grad, M_array, bias_grad)
        return output_grad, bias_grad, None


def add_expert_bias(y: torch.Tensor, bias: torch.Tensor, M_array: torch.Tensor) -> torch.Tensor:
    return _ExpertBias.apply(y, bias, M_array)


class _UpProjectionSwiglu(torch.autograd.Function):
    """a_e = swiglu_packed(x_e @ W_e^T) with the activation fused into the GEMM epilogue. The pre-activation h is
    kept (bf16) for the backward, which is swiglu-backward followed by the two grouped GEMMs."""

    @staticmethod
    @ensure_contiguous
    def forward(
        ctx, x: torch.Tensor, weight: torch.Tensor, M_array: torch.Tensor, N_array: torch.Tensor, K_array: torch.Tensor,
        grad_enabled: bool, bias: torch.Tensor | None = None,
    ) -> torch.Tensor:  # fmt: skip
        _, N, K = weight.size()
        assert N % 16 == 0
        assert K % 8 == 0
        R = x.size(0)
        # needs_input_grad only says that an input requires grad; under no_grad / inference_mode no backward will
        # follow (grad mode is always off inside forward, so the caller passes what it was outside)
        needs_backward = grad_enabled and any(ctx.needs_input_grad)
        h = torch.empty(R, N, device=x.device, dtype=x.dtype) if needs_backward else None
        act = torch.empty(R, N // 2, device=x.device, dtype=x.dtype)
        grouped_gemm_swiglu_cuda(x, weight, M_array, h, act, bias)
        if needs_backward:
            ctx.save_for_backward(x, weight, h, M_array, K_array, N_array)
        return act

    @staticmethod
    @ensure_contiguous
    def backward(ctx, act_grad: torch.Tensor) -> tuple[torch.Tensor | None]:
        from ...ops.swiglu.cuda_implementation import swiglu_backward_cuda

        x, weight, h, M_array, K_array, N_array = ctx.saved_tensors
        h_grad = torch.empty_like(h)
        up, gate = h.chunk(2, dim=-1)
        up_grad, gate_grad = h_grad.chunk(2, dim=-1)
        swiglu_backward_cuda(
            gate=gate, up=up, output_grad=act_grad, gate_grad=gate_grad, up_grad=up_grad, BLOCK_SIZE=1024
        )
        _, N, K = weight.size()
        x_grad = weight_grad = bias_grad = None
        if ctx.needs_input_grad[0]:
            x_grad = _expert_gemm(
                h_grad, weight, M_array, K_array, N_array, x.size(), "M", 0, K, N,
                is_A_transposed=False, is_B_transposed=False,
            )
        if ctx.needs_input_grad[1]:
            weight_grad = _expert_gemm(
                h_grad, x, N_array, K_array, M_array, weight.size(), "K", N, K, 0,
                is_A_transposed=True, is_B_transposed=False,
            )
        if len(ctx.needs_input_grad) > 6 and ctx.needs_input_grad[6]:
            bias_grad = torch.empty(weight.size(0), N, device=h_grad.device, dtype=h_grad.dtype)
            expert_bias_grad_cuda(h_grad, M_array, bias_grad)
        return (x_grad, weight_grad, None, None, None, None, bias_grad)[: len(ctx.needs_input_grad)]


class _SwigluExperts(torch.autograd.Function):
    """Both projections of a SwiGLU expert layer on grouped rows, o_e = swiglu_packed(x_e @ W1_e^T + b1_e) @ W2_e^T + b2_e,
    as one autograd node, so that the backward can keep the activation's gradient inside the second projection's input
    gradient: d_h comes out of one kernel (fma_grouped_gemm_swiglu_bwd) instead of a GEMM that writes d_a and an
    element-wise pass that reads it back. Same values, bit for bit, as _UpProjectionSwiglu followed by _GroupedGemmExperts."""

    @staticmethod
    @ensure_contiguous
    def forward(
        ctx, x: torch.Tensor, weight1: torch.Tensor, bias1: torch.Tensor | None, weight2: torch.Tensor,
        bias2: torch.Tensor | None, M_array: torch.Tensor, N1_array: torch.Tensor, K1_array: torch.Tensor,
        N2_array: torch.Tensor, K2_array: torch.Tensor, grad_enabled: bool,
    ) -> torch.Tensor:  # fmt: skip
        _, N1, K1 = weight1.size()
        _, N2, K2 = weight2.size()
        assert N1 % 16 == 0 and K1 % 8 == 0 and N2 % 8 == 0 and K2 == N1 // 2
        R = x.size(0)
        needs_backward = grad_enabled and any(ctx.needs_input_grad[:5])
        h = torch.empty(R, N1, device=x.device, dtype=x.dtype) if needs_backward else None
        act = torch.empty(R, K2, device=x.device, dtype=x.dtype)
        grouped_gemm_swiglu_cuda(x, weight1, M_array, h, act, bias1)
        output = _expert_gemm(
            act, weight2, M_array, N2_array, K2_array, (R, N2), "M", 0, N2, K2, is_A_transposed=False, is_B_transposed=True,
            bias=bias2,
        )
        if needs_backward:
            ctx.save_for_backward(x, weight1, weight2, h, act, M_array, N1_array, K1_array, N2_array, K2_array)
        ctx.has_bias = (bias1 is not None, bias2 is not None)
        return output

    @staticmethod
    @ensure_contiguous
    def backward(ctx, output_grad: torch.Tensor) -> tuple[torch.Tensor | None]:
        x, weight1, weight2, h, act, M_array, N1_array, K1_array, N2_array, K2_array = ctx.saved_tensors
        _, N1, K1 = weight1.size()
        _, N2, K2 = weight2.size()
        x_grad = weight1_grad = bias1_grad = weight2_grad = bias2_grad = None
        if ctx.needs_input_grad[3]:
            weight2_grad = _expert_gemm(
                output_grad, act, N2_array, K2_array, M_array, weight2.size(), "K", N2, K2, 0,
                is_A_transposed=True, is_B_transposed=False,
            )
        if ctx.has_bias[1] and ctx.needs_input_grad[4]:
            bias2_grad = torch.empty(weight2.size(0), N2, device=output_grad.device, dtype=output_grad.dtype)
            expert_bias_grad_cuda(output_grad, M_array, bias2_grad)
        if any(ctx.needs_input_grad[:3]):
            # d_h = backward of the activation at h applied to output_grad_e @ W2_e, in the GEMM's epilogue
            h_grad = torch.empty_like(h)
            grouped_gemm_swiglu_bwd_cuda(output_grad, weight2, h, M_array, h_grad)
            if ctx.needs_input_grad[0]:
                x_grad = _expert_gemm(
                    h_grad, weight1, M_array, K1_array, N1_array, x.size(), "M", 0, K1, N1,
                    is_A_transposed=False, is_B_transposed=False,
                )
            if ctx.needs_input_grad[1]:
                weight1_grad = _expert_gemm(
                    h_grad, x, N1_array, K1_array, M_array, weight1.size(), "K", N1, K1, 0,
                    is_A_transposed=True, is_B_transposed=False,
                )
            if ctx.has_bias[0] and ctx.needs_input_grad[2]:
                bias1_grad = torch.empty(weight1.size(0), N1, device=h_grad.device, dtype=h_grad.dtype)
                expert_bias_grad_cuda(h_grad, M_array, bias1_grad)
        return x_grad, weight1_grad, bias1_grad, weight2_grad, bias2_grad, None, None, None, None, None, None


def swiglu_experts(
    x: torch.Tensor, weight1: torch.Tensor, bias1: torch.Tensor | None, weight2: torch.Tensor, bias2: torch.Tensor | None,
    M_array: torch.Tensor, N1_array: torch.Tensor, K1_array: torch.Tensor, N2_array: torch.Tensor, K2_array: torch.Tensor,
) -> torch.Tensor:  # fmt: skip
    return _SwigluExperts.apply(
        x, weight1, bias1, weight2, bias2, M_array, N1_array, K1_array, N2_array, K2_array, torch.is_grad_enabled()
    )


class _GatheredUpProjection(torch.autograd.Function):
    """The first expert projection on tokens instead of grouped rows: y_i = x[perm[i] // top_k] @ W_e^T (+ bias_e), with
    swiglu_packed applied in the epilogue if `swiglu`. The rows are gathered inside the operand loads of the forward GEMM
    and of the weight-gradient GEMM, so the [T * top_k, H] buffer of grouped rows never exists; the backward returns the
    gradient per token."""

    @staticmethod
    @ensure_contiguous
    def forward(
        ctx, x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, perm: torch.Tensor, inv: torch.Tensor,
        M_array: torch.Tensor, N_array: torch.Tensor, K_array: torch.Tensor, top_k: int, swiglu: bool, grad_enabled: bool,
    ) -> torch.Tensor:  # fmt: skip
        _, N, K = weight.size()
        assert N % (16 if swiglu else 8) == 0 and K % 8 == 0
        R = perm.numel()
        needs_backward = grad_enabled and any(ctx.needs_input_grad[:3])
        if swiglu:
            h = torch.empty(R, N, device=x.device, dtype=x.dtype) if needs_backward else None
            output = torch.empty(R, N // 2, device=x.device, dtype=x.dtype)
            grouped_gemm_gathered_cuda(x, perm, top_k, weight, bias, M_array, h, output)
        else:
            h = None
            output = torch.empty(R, N, device=x.device, dtype=x.dtype)
            grouped_gemm_gathered_cuda(x, perm, top_k, weight, bias, M_array, output, None)
        if needs_backward:
            ctx.save_for_backward(x, weight, h, perm, inv, M_array, K_array, N_array)
        ctx.top_k = top_k
        ctx.has_bias = bias is not None
        return output

    @staticmethod
    @ensure_contiguous
    def backward(ctx, output_grad: torch.Tensor) -> tuple[torch.Tensor | None]:
        from ...ops.swiglu.cuda_implementation import swiglu_backward_cuda

        x, weight, h, perm, inv, M_array, K_array, N_array = ctx.saved_tensors
        _, N, K = weight.size()
        if h is not None:
            h_grad = torch.empty_like(h)
            up, gate = h.chunk(2, dim=-1)
            up_grad, gate_grad = h_grad.chunk(2, dim=-1)
            swiglu_backward_cuda(
                gate=gate, up=up, output_grad=output_grad, gate_grad=gate_grad, up_grad=up_grad, BLOCK_SIZE=1024
            )
        else:
            h_grad = output_grad
        x_grad = weight_grad = bias_grad = None
        if ctx.needs_input_grad[0]:
            grouped_grad = _expert_gemm(
                h_grad, weight, M_array, K_array, N_array, (h_grad.size(0), K), "M", 0, K, N,
                is_A_transposed=False, is_B_transposed=False,
            )
            x_grad = torch.empty_like(x)
            combine_cuda(grouped_grad, inv, None, ctx.top_k, x_grad)
        if ctx.needs_input_grad[1]:
            weight_grad = torch.empty_like(weight)
            grouped_gemm_gathered_wgrad_cuda(h_grad, x, perm, ctx.top_k, M_array, weight_grad)
        if ctx.has_bias and ctx.needs_input_grad[2]:
            bias_grad = torch.empty(weight.size(0), N, device=h_grad.device, dtype=h_grad.dtype)
            expert_bias_grad_cuda(h_grad, M_array, bias_grad)
        return x_grad, weight_grad, bias_grad, None, None, None, None, None, None, None, None


class _GatheredSwigluExperts(torch.autograd.Function):
    """_SwigluExperts on tokens instead of grouped rows: o_e = swiglu_packed(x[perm[i] // top_k] @ W1_e^T + b1_e) @ W2_e^T +
    b2_e. The first projection and its weight gradient gather the rows inside their operand loads, so a training step
    neither writes nor keeps the [T * top_k, H] buffer of grouped rows; the input gradient is summed per token here.
    Same values, bit for bit, as gather_rows followed by _SwigluExperts."""

    @staticmethod
    @ensure_contiguous
    def forward(
        ctx, x: torch.Tensor, weight1: torch.Tensor, bias1: torch.Tensor | None, weight2: torch.Tensor,
        bias2: torch.Tensor | None, perm: torch.Tensor, inv: torch.Tensor, M_array: torch.Tensor, N1_array: torch.Tensor,
        K1_array: torch.Tensor, N2_array: torch.Tensor, K2_array: torch.Tensor, top_k: int, grad_enabled: bool,
    ) -> torch.Tensor:  # fmt: skip
        _, N1, K1 = weight1.size()
        _, N2, K2 = weight2.size()
        assert N1 % 16 == 0 and K1 % 8 == 0 and N2 % 8 == 0 and K2 == N1 // 2
        R = perm.numel()
        needs_backward = grad_enabled and any(ctx.needs_input_grad[:5])
        h = torch.empty(R, N1, device=x.device, dtype=x.dtype) if needs_backward else None
        act = torch.empty(R, K2, device=x.device, dtype=x.dtype)
        grouped_gemm_gathered_cuda(x, perm, top_k, weight1, bias1, M_array, h, act)
        output = _expert_gemm(
            act, weight2, M_array, N2_array, K2_array, (R, N2), "M", 0, N2, K2, is_A_transposed=False, is_B_transposed=True,
            bias=bias2,
        )
        if needs_backward:
            ctx.save_for_backward(x, weight1, weight2, h, act, perm, inv, M_array, N1_array, K1_array, N2_array, K2_array)
        ctx.has_bias = (bias1 is not None, bias2 is not None)
        ctx.top_k = top_k
        return output

    @staticmethod
    @ensure_contiguous
    def backward(ctx, output_grad: torch.Tensor) -> tuple[torch.Tensor | None]:
        x, weight1, weight2, h, act, perm, inv, M_array, N1_array, K1_array, N2_array, K2_array = ctx.saved_tensors
        _, N1, K1 = weight1.size()
        _, N2, K2 = weight2.size()
        x_grad = weight1_grad = bias1_grad = weight2_grad = bias2_grad = None
        if ctx.needs_input_grad[3]:
            weight2_grad = _expert_gemm(
                output_grad, act, N2_array, K2_array, M_array, weight2.size(), "K", N2, K2, 0,
                is_A_transposed=True, is_B_transposed=False,
            )
        if ctx.has_bias[1] and ctx.needs_input_grad[4]:
            bias2_grad = torch.empty(weight2.size(0), N2, device=output_grad.device, dtype=output_grad.dtype)
            expert_bias_grad_cuda(output_grad, M_array, bias2_grad)
        if any(ctx.needs_input_grad[:3]):
            h_grad = torch.empty_like(h)
            grouped_gemm_swiglu_bwd_cuda(output_grad, weight2, h, M_array, h_grad)
            if ctx.needs_input_grad[0]:
                grouped_grad = _expert_gemm(
                    h_grad, weight1, M_array, K1_array, N1_array, (h_grad.size(0), K1), "M", 0, K1, N1,
                    is_A_transposed=False, is_B_transposed=False,
                )
                x_grad = torch.empty_like(x)
                combine_cuda(grouped_grad, inv, None, ctx.top_k, x_grad)
            if ctx.needs_input_grad[1]:
                weight1_grad = torch.empty_like(weight1)
                grouped_gemm_gathered_wgrad_cuda(h_grad, x, perm, ctx.top_k, M_array, weight1_grad)
            if ctx.has_bias[0] and ctx.needs_input_grad[2]:
                bias1_grad = torch.empty(weight1.size(0), N1, device=h_grad.device, dtype=h_grad.dtype)
                expert_bias_grad_cuda(h_grad, M_array, bias1_grad)
        return (x_grad, weight1_grad, bias1_grad, weight2_grad, bias2_grad) + (None,) * 9


def gathered_swiglu_experts(
    x: torch.Tensor, weight1: torch.Tensor, bias1: torch.Tensor | None, weight2: torch.Tensor, bias2: torch.Tensor | None,
    perm: torch.Tensor, inv: torch.Tensor, M_array: torch.Tensor, N1_array: torch.Tensor, K1_array: torch.Tensor,
    N2_array: torch.Tensor, K2_array: torch.Tensor, top_k: int,
) -> torch.Tensor:  # fmt: skip
    return _GatheredSwigluExperts.apply(
        x, weight1, bias1, weight2, bias2, perm, inv, M_array, N1_array, K1_array, N2_array, K2_array, top_k,
        torch.is_grad_enabled(),
    )


def gathered_up_projection_experts(
    x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, perm: torch.Tensor, inv: torch.Tensor,
    M_array: torch.Tensor, N_array: torch.Tensor, K_array: torch.Tensor, top_k: int, swiglu: bool,
) -> torch.Tensor:  # fmt: skip
    return _GatheredUpProjection.apply(
        x, weight, bias, perm, inv, M_array, N_array, K_array, top_k, swiglu, torch.is_grad_enabled()
    )


def can_gather_inside_gemm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None) -> bool:
    """the size and type limits of fma_grouped_gemm_gathered"""
    _, N, K = weight.size()
    return (
        x.is_cuda
        and x.dtype in (torch.bfloat16, torch.float16)
        and weight.dtype == x.dtype
        and (bias is None or bias.dtype == x.dtype)
        and N % 16 == 0
        and K % 8 == 0
        and N < (1 << 23)
        and K < (1 << 21)
        and 0 < x.size(0) * K * 2 < (1 << 31)
    )


# ---- the reference's padded grouping interface -------------------------------------------------------
# The MoE module above does not pad (the grouped GEMM masks ragged group edges). These keep the call signatures of
# fma/modules/moe/cuda_implementation/__init__.py:83-280 for code that calls them directly; the row movement itself is
# the dispatch / gather / combine kernels with a destination index that includes the padding offsets.


@torch.no_grad()
def _get_expert_padding_offset(
    expert_frequency: torch.Tensor, E: int, pad_to_multiple_of: int
) -> tuple[torch.Tensor, torch.Tensor]:
    """pad[e] = p - (M_e mod p), in [1, p] (an expert whose count is a multiple of p still gets p rows of padding);
    returns (M_e + pad[e] as uint32[E], [0, cumsum(pad)] as int64[E + 1])
    (fma/modules/moe/cuda_implementation/__init__.py:83-104, padded_expert_frequency_kernel.py:14-24)."""
    assert expert_frequency.numel() == E
    frequency = expert_frequency.to(torch.int64)
    padding = pad_to_multiple_of - frequency % pad_to_multiple_of
    padded_expert_frequency = (frequency + padding).to(torch.uint32)
    expert_padding_offset = torch.cat([padding.new_zeros(1), padding.cumsum(-1)])
    return padded_expert_frequency, expert_padding_offset


def _padded_row_of_slot(
    expert_padding_offset: torch.Tensor | None, sorted_idxs: torch.Tensor, scattered_idxs: torch.Tensor
) -> torch.Tensor:
    """int32[R]: the (padded) grouped row that holds slot s. sorted_idxs[i] is the expert of grouped row i,
    scattered_idxs[i] the slot it comes from (group_kernel.py:26-74: row i of expert e lands at i + offset[e])."""
    R = scattered_idxs.numel()
    rows = torch.arange(R, device=scattered_idxs.device, dtype=torch.int64)
    if expert_padding_offset is not None:
        rows = rows + expert_padding_offset.to(torch.int64)[sorted_idxs.long()]
    row_of_slot = torch.empty(R, device=scattered_idxs.device, dtype=torch.int32)
    row_of_slot[scattered_idxs.long()] = rows.to(torch.int32)
    return row_of_slot


class _GroupWithPadding(torch.autograd.Function):
    @staticmethod
    @ensure_contiguous
    def forward(
        ctx,
        x: torch.Tensor,
        expert_frequency: torch.Tensor,
        sorted_idxs: torch.Tensor,
        scattered_idxs: torch.Tensor,
        top_k: int,
        pad_to_multiple_of: int,
    ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor | None]:
        assert x.dim() == 2
        T, H = x.size()
        E = expert_frequency.size(0)
        assert H % 8 == 0

        if pad_to_multiple_of == 1:
            output = torch.empty(T * top_k, H, device=x.device, dtype=x.dtype)
            padded_expert_frequency = expert_frequency
            expert_padding_offset = None
        else:
            # the data-independent upper bound on the padded row count, zero-filled (the reference's shape)
            rows = (-(-(T * top_k) // pad_to_multiple_of) + E) * pad_to_multiple_of
            output = torch.zeros(rows, H, device=x.device, dtype=x.dtype)
            padded_expert_frequency, expert_padding_offset = _get_expert_padding_offset(
                expert_frequency=expert_frequency, E=E, pad_to_multiple_of=pad_to_multiple_of
            )

        row_of_slot = _padded_row_of_slot(expert_padding_offset, sorted_idxs, scattered_idxs)
        dispatch_rows_cuda(x, row_of_slot, top_k, output)

        ctx.save_for_backward(row_of_slot)
        ctx.T = T
        ctx.K = top_k
        return output, padded_expert_frequency, expert_padding_offset

    @staticmethod
    @ensure_contiguous
    def backward(ctx, output_grad: torch.Tensor, _: torch.Tensor, __: torch.Tensor) -> tuple[torch.Tensor | None]:
        (row_of_slot,) = ctx.saved_tensors
        # fp32 accumulation over the top_k rows of a token in a fixed order (the reference: fp32 atomics, then a cast)
        x_grad = torch.empty(ctx.T, output_grad.size(-1), device=output_grad.device, dtype=output_grad.dtype)
        combine_cuda(output_grad, row_of_slot, None, ctx.K, x_grad)
        return x_grad, *[None] * 5


class _UngroupWithPadding(torch.autograd.Function):
    @staticmethod
    @ensure_contiguous
    def forward(
        ctx,
        x: torch.Tensor,
        expert_padding_offset: torch.Tensor | None,
        sorted_idxs: torch.Tensor,
        scattered_idxs: torch.Tensor,
        top_k: int,
        num_tokens: int,
        pad_to_multiple_of: int,
    ) -> torch.Tensor:
        assert x.dim() == 2
        H = x.size(-1)
        assert H % 8 == 0
        output = torch.empty(num_tokens, top_k, H, device=x.device, dtype=x.dtype)

        row_of_slot = _padded_row_of_slot(expert_padding_offset, sorted_idxs, scattered_idxs)
        gather_rows_cuda(x, row_of_slot, 1, output.view(num_tokens * top_k, H))

        ctx.save_for_backward(row_of_slot)
        ctx.x_shape = x.size()
        ctx.pad_to_multiple_of = pad_to_multiple_of
        return output

    @staticmethod
    @ensure_contiguous
    def backward(ctx, output_grad: torch.Tensor) -> tuple[torch.Tensor | None]:
        (row_of_slot,) = ctx.saved_tensors
        T, K, H = output_grad.size()
        x_grad = (torch.empty if ctx.pad_to_multiple_of == 1 else torch.zeros)(
            *ctx.x_shape, device=output_grad.device, dtype=output_grad.dtype
        )
        dispatch_rows_cuda(output_grad.view(T * K, H), row_of_slot, 1, x_grad)
        return x_grad, *[None] * 6


def group_with_padding(
    x: torch.Tensor,
    expert_frequency: torch.Tensor,
    sorted_idxs: torch.Tensor,
    scattered_idxs: torch.Tensor,
    top_k: int,
    pad_to_multiple_of: int = 1,
) -> torch.Tensor:
    return _GroupWithPadding.apply(x, expert_frequency, sorted_idxs, scattered_idxs, top_k, pad_to_multiple_of)


def ungroup_with_padding(
    x: torch.Tensor,
    expert_padding_offset: torch.Tensor,
    sorted_idxs: torch.Tensor,
    scattered_idxs: torch.Tensor,
    top_k: int,
    num_tokens: int,
    pad_to_multiple_of: int,
) -> torch.Tensor:
    return _UngroupWithPadding.apply(
        x, expert_padding_offset, sorted_idxs, scattered_idxs, top_k, num_tokens, pad_to_multiple_of
    )


def gather_rows(x: torch.Tensor, perm: torch.Tensor, inv: torch.Tensor, top_k: int) -> torch.Tensor:
    return _GatherRows.apply(x, perm, inv, top_k)


def combine(o: torch.Tensor, gates: torch.Tensor, inv: torch.Tensor) -> torch.Tensor:
    return _Combine.apply(o, gates, inv)


def grouped_gemm_experts(
    x: torch.Tensor, weight: torch.Tensor, M_array: torch.Tensor, N_array: torch.Tensor, K_array: torch.Tensor,
    bias: torch.Tensor | None = None,
) -> torch.Tensor:  # fmt: skip
    """y_e = x_e @ W_e^T + bias_e. The 16-bit kernel adds the bias in its epilogue (within its size limits); otherwise
    it is a pass of its own over the fresh output."""
    if bias is None:
        return _GroupedGemmExperts.apply(x, weight, M_array, N_array, K_array)
    _, N, K = weight.size()
    if x.dtype in (torch.bfloat16, torch.float16) and bias.dtype == x.dtype and N < (1 << 23) and K < (1 << 21):
        return _GroupedGemmExperts.apply(x, weight, M_array, N_array, K_array, bias)
    return add_expert_bias(_GroupedGemmExperts.apply(x, weight, M_array, N_array, K_array), bias, M_array)


def up_projection_swiglu_experts(
    x: torch.Tensor, weight: torch.Tensor, M_array: torch.Tensor, N_array: torch.Tensor, K_array: torch.Tensor,
    bias: torch.Tensor | None = None,
) -> torch.Tensor:  # fmt: skip
    return _UpProjectionSwiglu.apply(x, weight, M_array, N_array, K_array, torch.is_grad_enabled(), bias)
