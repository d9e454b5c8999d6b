"""`swiglu_forward_cuda` / `swiglu_backward_cuda` custom ops: same names, arguments and mutation contract as the
reference's stubs (fma/ops/swiglu/cuda_implementation/__init__.py:16-30), bound to fma_swiglu_forward /
fma_swiglu_backward of libfma_hip.so. Unlike the reference's CUDA kernels they accept row-strided operands (the
reference needs its Triton kernels for that, fma/ops/swiglu/triton_implementation/forward.py:49-66)."""

import torch
from torch.library import custom_op

from ... import _lib
from ...constants import LIBRARY_NAME


def _rows_view(t: torch.Tensor) -> tuple[int, int, int] | None:
    """(rows, cols, row_stride) if `t` can be addressed as rows of `cols` contiguous elements, else None."""
    if t.dim() == 0:
        return 1, 1, 1
    cols = t.size(-1)
    if t.numel() == 0:
        return 0, cols, max(cols, 1)
    if cols != 1 and t.stride(-1) != 1:
        return None
    rows = t.numel() // cols
    row_stride = None
    expected = 0
    for d in range(t.dim() - 2, -1, -1):
        if t.size(d) == 1:
            continue
        if row_stride is None:
            row_stride = t.stride(d)
        elif t.stride(d) != expected:
            return None
        expected = t.stride(d) * t.size(d)
    if row_stride is None:
        row_stride = cols
    if row_stride < cols:
        return None
    return rows, cols, row_stride


def _as_rows(t: torch.Tensor, writable: bool) -> tuple[torch.Tensor, int, int, int]:
    view = _rows_view(t)
    if view is None:
        assert not writable, "output tensors must be addressable as rows of contiguous elements"
        t = t.contiguous()
        view = _rows_view(t)
    return (t,) + view


@custom_op(f"{LIBRARY_NAME}::swiglu_forward_cuda", mutates_args={"output"})
def swiglu_forward_cuda(gate: torch.Tensor, up: torch.Tensor, output: torch.Tensor, BLOCK_SIZE: int) -> None:
    _lib.require_gpu(gate, up, output)
    assert gate.shape == up.shape == output.shape
    assert gate.dtype == up.dtype == output.dtype
    gate, rows, cols, gs = _as_rows(gate, False)
    up, _, _, us = _as_rows(up, False)
    output, _, _, os_ = _as_rows(output, True)
    with torch.cuda.device(gate.device):
        rc = _lib.load().fma_swiglu_forward(
            gate.data_ptr(), up.data_ptr(), output.data_ptr(), rows, cols, gs, us, os_, _lib.dtype_code(gate.dtype),
            _lib.current_stream(gate.device),
        )
    _lib.check(rc, "swiglu_forward_cuda")


@custom_op(f"{LIBRARY_NAME}::swiglu_backward_cuda", mutates_args={"gate_grad", "up_grad"})
def swiglu_backward_cuda(
    gate: torch.Tensor,
    up: torch.Tensor,
    output_grad: torch.Tensor,
    gate_grad: torch.Tensor,
    up_grad: torch.Tensor,
    BLOCK_SIZE: int,
) -> None:
    _lib.require_gpu(gate, up, output_grad, gate_grad, up_grad)
    assert gate.shape == up.shape == output_grad.shape == gate_grad.shape == up_grad.shape
    assert gate.dtype == up.dtype == output_grad.dtype == gate_grad.dtype == up_grad.dtype
    gate, rows, cols, gs = _as_rows(gate, False)
    up, _, _, us = _as_rows(up, False)
    output_grad, _, _, ds = _as_rows(output_grad, False)
    gate_grad, _, _, ggs = _as_rows(gate_grad, True)
    up_grad, _, _, ugs = _as_rows(up_grad, True)
    with torch.cuda.device(gate.device):
        rc = _lib.load().fma_swiglu_backward(
            gate.data_ptr(), up.data_ptr(), output_grad.data_ptr(), gate_grad.data_ptr(), up_grad.data_ptr(), rows,
            cols, gs, us, ds, ggs, ugs, _lib.dtype_code(gate.dtype), _lib.current_stream(gate.device),
        )
    _lib.check(rc, "swiglu_backward_cuda")
