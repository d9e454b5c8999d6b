"""`grouped_gemm`: one matrix product per group over operands that hold the groups back to back. Signature, defaults and
the two assertions follow fma/ops/grouped_gemm/__init__.py:11-46; the product is `fma_grouped_gemm` of libfma_hip.so."""

import torch

from ...utils import ensure_contiguous
from .cuda_implementation import grouped_gemm_cuda


@ensure_contiguous
def grouped_gemm(
    A: torch.Tensor, B: torch.Tensor, C: torch.Tensor | None,
    M_array: torch.Tensor, N_array: torch.Tensor, K_array: torch.Tensor,
    output_shape: tuple[int, int], alpha: float = 1, beta: float = 0,
    is_A_transposed: bool = False, is_B_transposed: bool = False, benchmark: bool = False,
) -> torch.Tensor:  # fmt: skip
    """D_e = alpha * op(A_e) @ op(B_e) for every group e; groups lie back to back in A, B and the result.

    A_e is stored [M_e, K_e], or [K_e, M_e] with is_A_transposed; B_e is stored [K_e, N_e], or [N_e, K_e] with
    is_B_transposed. M_array / N_array / K_array are uint32 device tensors with one entry per group and stay on the
    device. Like the reference, only beta == 0 without C exists. Returns a new tensor of `output_shape` in A's dtype.
    """
    assert beta == 0
    assert C is None

    result = A.new_empty(tuple(output_shape))
    sizes = dict(M_array=M_array, N_array=N_array, K_array=K_array)
    layout = dict(is_A_transposed=is_A_transposed, is_B_transposed=is_B_transposed)
    grouped_gemm_cuda(A=A, B=B, C=C, output=result, **sizes, **layout, alpha=alpha, beta=beta, benchmark=benchmark)
    return result
