"""`grouped_gemm_cuda` custom op: same name, arguments and mutation contract as the reference's stub
(fma/ops/grouped_gemm/cuda_implementation/__init__.py:15-30), bound to fma_grouped_gemm of libfma_hip.so."""

import torch
from torch.library import custom_op

from ... import _lib
from ...constants import LIBRARY_NAME


def _launch(A, B, output, M_array, N_array, K_array, is_A_transposed, is_B_transposed, alpha) -> None:
    lib = _lib.load()
    if output.numel() == 0:
        return
    # An operand without elements (every group has M_e * K_e == 0, resp. K_e * N_e == 0) is never read, but the entry point
    # rejects NULL: any valid device address stands in for it.
    a_ptr = A.data_ptr() if A.numel() else output.data_ptr()
    b_ptr = B.data_ptr() if B.numel() else output.data_ptr()
    with torch.cuda.device(A.device):
        rc = lib.fma_grouped_gemm(
            a_ptr, b_ptr, output.data_ptr(), M_array.data_ptr(), N_array.data_ptr(), K_array.data_ptr(),
            M_array.numel(), int(is_A_transposed), int(is_B_transposed), float(alpha), _lib.dtype_code(A.dtype),
            _lib.current_stream(A.device),
        )
    _lib.check(rc, "grouped_gemm_cuda")


@custom_op(f"{LIBRARY_NAME}::grouped_gemm_cuda", mutates_args={"output"})
def grouped_gemm_cuda(
    A: torch.Tensor,
    B: torch.Tensor,
    C: torch.Tensor | None,
    output: torch.Tensor,
    M_array: torch.Tensor,
    N_array: torch.Tensor,
    K_array: torch.Tensor,
    is_A_transposed: bool,
    is_B_transposed: bool,
    alpha: float,
    beta: float,
    benchmark: bool,
) -> None:
    assert beta == 0 and C is None
    _lib.require_gpu(A, B, output, M_array, N_array, K_array)
    assert A.dtype == B.dtype == output.dtype
    for arr in (M_array, N_array, K_array):
        assert arr.dtype == torch.uint32 and arr.is_contiguous()
    assert M_array.numel() == N_array.numel() == K_array.numel()
    assert A.is_contiguous() and B.is_contiguous() and output.is_contiguous()

    _launch(A, B, output, M_array, N_array, K_array, is_A_transposed, is_B_transposed, alpha)

    if benchmark:
        # same report as the reference's benchmark flag (kernel.cu:335-351), with the real flop count
        flops = 2.0 * float(
            (M_array.to(torch.int64) * N_array.to(torch.int64) * K_array.to(torch.int64)).sum().item()
        )
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        iterations = 10
        start.record()
        for _ in range(iterations):
            _launch(A, B, output, M_array, N_array, K_array, is_A_transposed, is_B_transposed, alpha)
        stop.record()
        stop.synchronize()
        ms = start.elapsed_time(stop) / iterations
        print(f"grouped_gemm: {ms:.3f} ms, {flops / ms / 1e9:.1f} TFLOP/s")
