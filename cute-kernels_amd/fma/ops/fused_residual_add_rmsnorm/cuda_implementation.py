"""Custom ops over fma_fused_residual_add_rmsnorm_fwd / _bwd of libfma_hip.so. They take the argument lists of the
reference's fused_residual_add_rmsnorm_forward_triton / fused_residual_add_rmsnorm_backward_triton
(fma/ops/fused_residual_add_rmsnorm/triton_implementation/forward.py:64-102, backward.py:101-145)."""

import torch
from torch.library import custom_op

from ... import _lib
from ...constants import LIBRARY_NAME
from ...utils import get_num_elements_and_hidden_size


@custom_op(
    f"{LIBRARY_NAME}::fused_residual_add_rmsnorm_forward_cuda",
    mutates_args={"output", "added_x_residual", "rmsnorm_denominator"},
)
def fused_residual_add_rmsnorm_forward_cuda(
    x: torch.Tensor,
    residual: torch.Tensor,
    weight: torch.Tensor | None,
    output: torch.Tensor,
    eps: float,
    multiplier: float | None,
    added_x_residual: torch.Tensor,
    rmsnorm_denominator: torch.Tensor | None,
) -> None:
    _lib.require_gpu(x, residual, weight, output, added_x_residual, rmsnorm_denominator)
    B, H = get_num_elements_and_hidden_size(x)
    assert residual.size() == x.size() == output.size() == added_x_residual.size()
    assert residual.dtype == x.dtype == output.dtype == added_x_residual.dtype
    assert weight is None or (weight.dtype == x.dtype and weight.numel() == H)
    assert rmsnorm_denominator is None or (rmsnorm_denominator.dtype == torch.float32 and rmsnorm_denominator.numel() == B)
    for t in (x, residual, weight, output, added_x_residual, rmsnorm_denominator):
        assert t is None or t.is_contiguous()
    with torch.cuda.device(x.device):
        rc = _lib.load().fma_fused_residual_add_rmsnorm_fwd(
            x.data_ptr(), residual.data_ptr(), _lib.ptr(weight), output.data_ptr(), added_x_residual.data_ptr(),
            _lib.ptr(rmsnorm_denominator), B, H, eps, 1.0 if multiplier is None else multiplier,
            _lib.dtype_code(x.dtype), _lib.current_stream(x.device),
        )
    _lib.check(rc, "fused_residual_add_rmsnorm_forward_cuda")


@custom_op(
    f"{LIBRARY_NAME}::fused_residual_add_rmsnorm_backward_cuda",
    mutates_args={"x_grad", "residual_grad", "weight_grad"},
)
def fused_residual_add_rmsnorm_backward_cuda(
    added_x_residual: torch.Tensor,
    weight: torch.Tensor | None,
    output_grad: torch.Tensor,
    added_x_residual_grad: torch.Tensor | None,
    rmsnorm_denominator: torch.Tensor | None,
    x_grad: torch.Tensor,
    residual_grad: torch.Tensor,
    weight_grad: torch.Tensor | None,
    eps: float,
    multiplier: float | None,
) -> None:
    _lib.require_gpu(
        added_x_residual, weight, output_grad, added_x_residual_grad, rmsnorm_denominator, x_grad, residual_grad, weight_grad
    )
    B, H = get_num_elements_and_hidden_size(added_x_residual)
    for t in (output_grad, added_x_residual_grad, x_grad, residual_grad):
        assert t is None or (t.size() == added_x_residual.size() and t.dtype == added_x_residual.dtype)
    assert (weight is None) == (weight_grad is None)
    assert weight is None or (weight.dtype == added_x_residual.dtype and weight.numel() == H)
    assert weight_grad is None or (weight_grad.dtype == torch.float32 and weight_grad.numel() == H)
    assert rmsnorm_denominator is None or (rmsnorm_denominator.dtype == torch.float32 and rmsnorm_denominator.numel() == B)
    for t in (added_x_residual, weight, output_grad, added_x_residual_grad, rmsnorm_denominator, x_grad, residual_grad, weight_grad):
        assert t is None or t.is_contiguous()
    lib = _lib.load()
    with torch.cuda.device(added_x_residual.device):
        # per-workgroup partial weight gradients; scratch owned by this call
        nbytes = lib.fma_fused_residual_add_rmsnorm_bwd_workspace_bytes(B, H) if weight is not None else 0
        workspace = torch.empty(max(nbytes, 4), dtype=torch.uint8, device=added_x_residual.device)
        rc = lib.fma_fused_residual_add_rmsnorm_bwd(
            added_x_residual.data_ptr(), _lib.ptr(weight), output_grad.data_ptr(), _lib.ptr(added_x_residual_grad),
            _lib.ptr(rmsnorm_denominator), x_grad.data_ptr(), residual_grad.data_ptr(), _lib.ptr(weight_grad), B, H, eps,
            1.0 if multiplier is None else multiplier, workspace.data_ptr(), nbytes,
            _lib.dtype_code(added_x_residual.dtype), _lib.current_stream(added_x_residual.device),
        )
    _lib.check(rc, "fused_residual_add_rmsnorm_backward_cuda")
