"""`swiglu(gate, up)` and `swiglu_packed(x)`: y = up * gate * sigmoid(gate), with gradients. Public names, keyword
arguments, defaults, the shape / dtype assertions and the ValueError for an unknown backend are those of
fma/ops/swiglu/__init__.py:15-164. A packed input holds [up | gate] along its last dimension (the reference's
`up, gate = x.chunk(2, dim=-1)`, :153). Both forms end in the same two strided HIP kernels (`fma_swiglu_forward`,
`fma_swiglu_backward`): the halves of a packed tensor are passed as views, never copied."""

import torch

from ...kernel_backend import KernelBackend, is_hip_kernel_backend
from ...math import divide_if_divisible
from ...utils import ensure_contiguous
from .cuda_implementation import swiglu_backward_cuda, swiglu_forward_cuda

_BLOCK_SIZE = 1024  # a launch-shape argument of the reference's stubs; the HIP kernels choose their own


def _require_hip(*kernel_backends: KernelBackend) -> None:
    for kernel_backend in kernel_backends:
        if not is_hip_kernel_backend(kernel_backend):
            raise ValueError(f"unexpected kernel_backend ({kernel_backend})")


def _forward(gate: torch.Tensor, up: torch.Tensor, output: torch.Tensor) -> torch.Tensor:
    swiglu_forward_cuda(gate=gate, up=up, output=output, BLOCK_SIZE=_BLOCK_SIZE)
    return output


def _backward(gate, up, output_grad, gate_grad, up_grad) -> None:
    swiglu_backward_cuda(
        gate=gate, up=up, output_grad=output_grad, gate_grad=gate_grad, up_grad=up_grad, BLOCK_SIZE=_BLOCK_SIZE
    )


class _Swiglu(torch.autograd.Function):
    """Two separate operands of one shape."""

    @staticmethod
    @ensure_contiguous
    def forward(ctx, gate: torch.Tensor, up: torch.Tensor, forward_backend, backward_backend) -> torch.Tensor:
        assert gate.size() == up.size(), "tensors gate and up should have same shape"
        assert gate.type() == up.type(), "tensors gate and up should have same dtype"
        _require_hip(forward_backend, backward_backend)
        ctx.save_for_backward(gate, up)
        return _forward(gate, up, torch.empty_like(gate))

    @staticmethod
    @ensure_contiguous
    def backward(ctx, output_grad: torch.Tensor):
        gate, up = ctx.saved_tensors
        grads = torch.empty_like(gate), torch.empty_like(up)
        _backward(gate, up, output_grad, *grads)
        return (*grads, None, None)


class _SwigluPacked(torch.autograd.Function):
    """One operand whose last dimension is [up | gate]; its gradient is written in the same packing."""

    @staticmethod
    @ensure_contiguous
    def forward(ctx, x: torch.Tensor, forward_backend, backward_backend) -> torch.Tensor:
        _require_hip(forward_backend, backward_backend)
        half = divide_if_divisible(x.size(-1), 2)
        up, gate = x.split(half, dim=-1)
        ctx.save_for_backward(x)
        return _forward(gate, up, x.new_empty(*x.shape[:-1], half))

    @staticmethod
    @ensure_contiguous
    def backward(ctx, output_grad: torch.Tensor):
        (x,) = ctx.saved_tensors
        half = x.size(-1) // 2
        x_grad = torch.empty_like(x)
        up, gate = x.split(half, dim=-1)
        up_grad, gate_grad = x_grad.split(half, dim=-1)
        _backward(gate, up, output_grad, gate_grad, up_grad)
        return x_grad, None, None


def swiglu(
    gate: torch.Tensor,
    up: torch.Tensor,
    *,
    kernel_backend_forward: KernelBackend = KernelBackend.cuda,
    kernel_backend_backward: KernelBackend = KernelBackend.cuda,
) -> torch.Tensor:
    """up * gate * sigmoid(gate) for two tensors of the same shape and dtype (fp32 arithmetic, output in their dtype).
    Both backends must name the HIP kernels (KernelBackend.cuda or .triton)."""
    return _Swiglu.apply(gate, up, kernel_backend_forward, kernel_backend_backward)


def swiglu_packed(
    x: torch.Tensor,
    *,
    kernel_backend_forward: KernelBackend = KernelBackend.triton,
    kernel_backend_backward: KernelBackend = KernelBackend.triton,
) -> torch.Tensor:
    """The same activation for x = [up | gate] along the last dimension (which must be even); the result has half
    that length. The defaults are the reference's (`triton`), served here by the HIP kernels."""
    return _SwigluPacked.apply(x, kernel_backend_forward, kernel_backend_backward)
