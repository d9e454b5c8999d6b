"""`fused_residual_add_rmsnorm`: residual = x * multiplier + residual; output = rms_norm(residual) * weight, both
returned, in one pass over the rows. Arguments, defaults, outputs, assertions and what is kept for the backward follow
fma/ops/fused_residual_add_rmsnorm/__init__.py:16-126; the work is done by `fma_fused_residual_add_rmsnorm_fwd` / `_bwd`
of libfma_hip.so where the reference calls its Triton kernels."""

import torch

from ...kernel_backend import KernelBackend, is_hip_kernel_backend
from ...utils import ensure_contiguous, get_num_elements_and_hidden_size
from .cuda_implementation import fused_residual_add_rmsnorm_backward_cuda, fused_residual_add_rmsnorm_forward_cuda


def _check_weight(weight: torch.Tensor | None, x: torch.Tensor) -> None:
    if weight is None:
        return
    assert weight.dim() == 1, "weight should be 1D"
    assert weight.size(-1) == x.size(-1), "hidden size for x and weight tensor is different"
    assert weight.type() == x.type(), "tensors weight and y should have same dtype"


class _FusedResidualAddRMSNorm(torch.autograd.Function):
    @staticmethod
    @ensure_contiguous
    def forward(ctx, x, residual, weight, eps, multiplier, memory_efficient, kernel_backend):
        if not is_hip_kernel_backend(kernel_backend):
            raise ValueError(f"unexpected kernel_backend ({kernel_backend})")
        _check_weight(weight, x)
        ctx.eps = torch.finfo(x.dtype).eps if eps is None else eps
        ctx.multiplier = multiplier

        rows, _ = get_num_elements_and_hidden_size(x)
        normed, stream = torch.empty_like(x), torch.empty_like(x)
        # 1 / rms of every row, kept for the backward unless the caller prefers to recompute it
        inverse_rms = None if memory_efficient else x.new_empty(rows, dtype=torch.float32)
        fused_residual_add_rmsnorm_forward_cuda(
            x=x, residual=residual, weight=weight, output=normed, eps=ctx.eps, multiplier=multiplier,
            added_x_residual=stream, rmsnorm_denominator=inverse_rms,
        )
        ctx.save_for_backward(stream, weight, inverse_rms)
        # an output that takes no part in the loss arrives as None instead of a tensor of zeros that would be read
        ctx.set_materialize_grads(False)
        return normed, stream

    @staticmethod
    @ensure_contiguous
    def backward(ctx, normed_grad, stream_grad):
        stream, weight, inverse_rms = ctx.saved_tensors
        if normed_grad is None and stream_grad is None:
            return (None,) * 7
        if normed_grad is None:
            normed_grad = torch.zeros_like(stream)
        x_grad, residual_grad = torch.empty_like(stream), torch.empty_like(stream)
        # fp32, fully written by the kernels (per-workgroup partial sums added in a fixed order): no zero-filling
        weight_grad = None if weight is None else torch.empty_like(weight, dtype=torch.float32)
        fused_residual_add_rmsnorm_backward_cuda(
            added_x_residual=stream, weight=weight, output_grad=normed_grad, added_x_residual_grad=stream_grad,
            rmsnorm_denominator=inverse_rms, x_grad=x_grad, residual_grad=residual_grad, weight_grad=weight_grad,
            eps=ctx.eps, multiplier=ctx.multiplier,
        )
        if weight_grad is not None:
            weight_grad = weight_grad.type_as(weight)
        return x_grad, residual_grad, weight_grad, None, None, None, None


def fused_residual_add_rmsnorm(
    x: torch.Tensor,
    residual: torch.Tensor,
    weight: torch.Tensor | None,
    eps: float | None,
    multiplier: float | None = None,
    memory_efficient: bool = False,
    kernel_backend: KernelBackend = KernelBackend.triton,
) -> tuple[torch.Tensor]:
    """Returns (normalised activations, updated residual stream), both shaped and typed like x.

    x, residual: tensors of one shape, rows along the last dimension. weight: 1-D scale of that length, or None.
    eps: added to the mean square; None takes the dtype's machine epsilon. multiplier: scales x before the add; None
    means 1. memory_efficient: do not keep the rows' 1 / rms for the backward. kernel_backend: the reference's default
    (`triton`) and `cuda` both run the HIP kernels; anything else raises ValueError.
    """
    return _FusedResidualAddRMSNorm.apply(x, residual, weight, eps, multiplier, memory_efficient, kernel_backend)
