"""`fused_residual_add_rmsnorm`: residual add and RMSNorm in one pass, returning the normalised activations and the
updated residual stream. Mirrors fma/ops/fused_residual_add_rmsnorm/__init__.py:16-126 (same arguments, same two outputs,
same saved tensors); the kernels are HIP kernels of libfma_hip.so instead of Triton.
"""

import torch

from ...kernel_backend import KernelBackend, is_hip_kernel_backend
from ...utils import ensure_contiguous, get_num_elements_and_hidden_size
from .cuda_implementation import fused_residual_add_rmsnorm_backward_cuda, fused_residual_add_rmsnorm_forward_cuda


class _FusedResidualAddRMSNorm(torch.autograd.Function):
    @staticmethod
    @ensure_contiguous
    def forward(
        ctx,
        x: torch.Tensor,
        residual: torch.Tensor,
        weight: torch.Tensor | None,
        eps: float | None,
        multiplier: float | None,
        memory_efficient: bool,
        kernel_backend: KernelBackend,
    ) -> tuple[torch.Tensor]:
        if not is_hip_kernel_backend(kernel_backend):
            raise ValueError(f"unexpected kernel_backend ({kernel_backend})")

        if weight is not None:
            assert weight.dim() == 1, "weight should be 1D"
            assert weight.size(-1) == x.size(-1), "hidden size for x and weight tensor is different"
            assert weight.type() == x.type(), "tensors weight and y should have same dtype"

        if eps is None:
            eps = torch.finfo(x.dtype).eps

        B, _ = get_num_elements_and_hidden_size(x)

        output = torch.empty_like(x)
        added_x_residual = torch.empty_like(x)
        rmsnorm_denominator = None if memory_efficient else torch.empty(B, device=x.device, dtype=torch.float32)

        fused_residual_add_rmsnorm_forward_cuda(
            x=x,
            residual=residual,
            weight=weight,
            output=output,
            eps=eps,
            multiplier=multiplier,
            added_x_residual=added_x_residual,
            rmsnorm_denominator=rmsnorm_denominator,
        )

        ctx.save_for_backward(added_x_residual, weight, rmsnorm_denominator)
        ctx.eps = eps
        ctx.multiplier = multiplier
        # an output that takes no part in the loss arrives as None instead of a tensor of zeros that would be read
        ctx.set_materialize_grads(False)

        return output, added_x_residual

    @staticmethod
    @ensure_contiguous
    def backward(
        ctx, output_grad: torch.Tensor | None, added_x_residual_grad: torch.Tensor | None
    ) -> tuple[torch.Tensor | None]:
        added_x_residual, weight, rmsnorm_denominator = ctx.saved_tensors
        if output_grad is None:
            if added_x_residual_grad is None:
                return (None,) * 7
            output_grad = torch.zeros_like(added_x_residual)
        x_grad = torch.empty_like(added_x_residual)
        residual_grad = torch.empty_like(added_x_residual)
        # fully written by the kernels (per-workgroup partial sums added in a fixed order), so no zero-filling
        weight_grad = None if weight is None else torch.empty_like(weight, dtype=torch.float32)

        fused_residual_add_rmsnorm_backward_cuda(
            added_x_residual=added_x_residual,
            weight=weight,
            output_grad=output_grad,
            added_x_residual_grad=added_x_residual_grad,
            rmsnorm_denominator=rmsnorm_denominator,
            x_grad=x_grad,
            residual_grad=residual_grad,
            weight_grad=weight_grad,
            eps=ctx.eps,
            multiplier=ctx.multiplier,
        )

        if weight_grad is not None:
            weight_grad = weight_grad.type_as(weight)

        return x_grad, residual_grad, weight_grad, *[None] * 4


def fused_residual_add_rmsnorm(
    x: torch.Tensor,
    residual: torch.Tensor,
    weight: torch.Tensor | None,
    eps: float | None,
    multiplier: float | None = None,
    memory_efficient: bool = False,
    kernel_backend: KernelBackend = KernelBackend.triton,
) -> tuple[torch.Tensor]:
    """fused residual add RMSNorm computation

    Args:
        x (torch.Tensor): input activation
        residual (torch.Tensor): residual activation
        weight (torch.Tensor | None): RMSNorm weight
        eps (float | None): epsilon
        multiplier (float | None, optional): if not None, pre-multiplies `x` with `multiplier`. Defaults to None.
        memory_efficient (bool, optional): memory efficient = False caches RMSNorm's denominator in the forward.
            Defaults to False.
        kernel_backend (KernelBackend, optional): any value but KernelBackend.torch runs the HIP kernels.

    Returns:
        tuple[torch.Tensor]: output activations, updated residual stream
    """
    return _FusedResidualAddRMSNorm.apply(x, residual, weight, eps, multiplier, memory_efficient, kernel_backend)
