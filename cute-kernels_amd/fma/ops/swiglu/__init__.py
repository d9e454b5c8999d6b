"""`swiglu` and `swiglu_packed`: y = up * gate * sigmoid(gate). Mirrors fma/ops/swiglu/__init__.py:15-164.

The packed form splits the last dimension as `up, gate = x.chunk(2, dim=-1)` (first half up, second half gate),
the reference's convention (fma/ops/swiglu/__init__.py:153). Both forms run the same strided HIP kernels, so the
halves of a packed tensor are never copied.
"""

import torch

from ...kernel_backend import KernelBackend, is_hip_kernel_backend
from ...math import divide_if_divisible
from ...utils import ensure_contiguous
from .cuda_implementation import swiglu_backward_cuda, swiglu_forward_cuda


def _check_backends(kernel_backend_forward: KernelBackend, kernel_backend_backward: KernelBackend) -> None:
    if not is_hip_kernel_backend(kernel_backend_forward):
        raise ValueError(f"unexpected kernel_backend ({kernel_backend_forward})")
    if not is_hip_kernel_backend(kernel_backend_backward):
        raise ValueError("unexpected kernel_backend")


class _Swiglu(torch.autograd.Function):
    @staticmethod
    @ensure_contiguous
    def forward(
        ctx,
        gate: torch.Tensor,
        up: torch.Tensor,
        kernel_backend_forward: KernelBackend,
        kernel_backend_backward: KernelBackend,
    ) -> torch.Tensor:
        assert gate.size() == up.size(), "tensors gate and up should have same shape"
        assert gate.type() == up.type(), "tensors gate and up should have same dtype"
        _check_backends(kernel_backend_forward, kernel_backend_backward)

        output = torch.empty_like(gate)
        swiglu_forward_cuda(gate=gate, up=up, output=output, BLOCK_SIZE=1024)

        ctx.save_for_backward(gate, up)
        return output

    @staticmethod
    @ensure_contiguous
    def backward(ctx, output_grad: torch.Tensor) -> tuple[torch.Tensor | None]:
        gate, up = ctx.saved_tensors
        gate_grad = torch.empty_like(gate)
        up_grad = torch.empty_like(up)

        swiglu_backward_cuda(
            gate=gate, up=up, output_grad=output_grad, gate_grad=gate_grad, up_grad=up_grad, BLOCK_SIZE=1024
        )

        return gate_grad, up_grad, None, None


class _SwigluPacked(torch.autograd.Function):
    @staticmethod
    @ensure_contiguous
    def forward(
        ctx,
        x: torch.Tensor,
        kernel_backend_forward: KernelBackend = KernelBackend.triton,
        kernel_backend_backward: KernelBackend = KernelBackend.triton,
    ) -> torch.Tensor:
        _check_backends(kernel_backend_forward, kernel_backend_backward)
        ctx.save_for_backward(x)

        output = torch.empty(*x.size()[:-1], divide_if_divisible(x.size(-1), 2), device=x.device, dtype=x.dtype)
        up, gate = x.chunk(2, dim=-1)

        swiglu_forward_cuda(gate=gate, up=up, output=output, BLOCK_SIZE=1024)

        return output

    @staticmethod
    @ensure_contiguous
    def backward(ctx, output_grad: torch.Tensor) -> tuple[torch.Tensor | None]:
        x: torch.Tensor = ctx.saved_tensors[0]
        x_grad = torch.empty_like(x)

        up, gate = x.chunk(2, dim=-1)
        up_grad, gate_grad = x_grad.chunk(2, dim=-1)

        swiglu_backward_cuda(
            gate=gate, up=up, output_grad=output_grad, gate_grad=gate_grad, up_grad=up_grad, BLOCK_SIZE=1024
        )

        return x_grad, None, None


def swiglu(
    gate: torch.Tensor,
    up: torch.Tensor,
    *,
    kernel_backend_forward: KernelBackend = KernelBackend.cuda,
    kernel_backend_backward: KernelBackend = KernelBackend.cuda,
) -> torch.Tensor:
    """computes swiglu activation as `up` * `gate` * sigmoid(`gate`)

    Args:
        gate (torch.Tensor): `gate` activation tensor
        up (torch.Tensor): `up` activation tensor
        kernel_backend_forward (KernelBackend, optional): KernelBackend.cuda (the HIP kernel).
        kernel_backend_backward (KernelBackend, optional): KernelBackend.cuda (the HIP kernel).

    Returns:
        torch.Tensor: output tensor
    """
    return _Swiglu.apply(gate, up, kernel_backend_forward, kernel_backend_backward)


def swiglu_packed(
    x: torch.Tensor,
    *,
    kernel_backend_forward: KernelBackend = KernelBackend.triton,
    kernel_backend_backward: KernelBackend = KernelBackend.triton,
) -> torch.Tensor:
    """computes swiglu activation by splitting the tensor `x` into 2 parts: up (first half) and gate (second half)

    Args:
        x (torch.Tensor): input activation, last dimension even
        kernel_backend_forward (KernelBackend, optional): any value but KernelBackend.torch runs the HIP kernel.
        kernel_backend_backward (KernelBackend, optional): any value but KernelBackend.torch runs the HIP kernel.

    Returns:
        torch.Tensor: output tensor
    """
    return _SwigluPacked.apply(x, kernel_backend_forward, kernel_backend_backward)
