"""`grouped_gemm`: one GEMM per group over ragged, packed operands. Mirrors fma/ops/grouped_gemm/__init__.py:11-46."""

import torch

from ...utils import ensure_contiguous
from .cuda_implementation import grouped_gemm_cuda


@ensure_contiguous
def grouped_gemm(
    A: torch.Tensor,
    B: torch.Tensor,
    C: torch.Tensor | None,
    M_array: torch.Tensor,
    N_array: torch.Tensor,
    K_array: torch.Tensor,
    output_shape: tuple[int, int],
    alpha: float = 1,
    beta: float = 0,
    is_A_transposed: bool = False,
    is_B_transposed: bool = False,
    benchmark: bool = False,
) -> torch.Tensor:
    """D_e = alpha * op(A_e) @ op(B_e) for every group e; groups are packed back to back in A, B and the output.

    is_A_transposed=False: A_e is stored [M_e, K_e]; True: [K_e, M_e].
    is_B_transposed=True:  B_e is stored [N_e, K_e]; False: [K_e, N_e].
    M_array / N_array / K_array are uint32 device tensors (one entry per group); they are never copied to the host.
    """
    assert beta == 0
    assert C is None

    output = torch.empty(*output_shape, device=A.device, dtype=A.dtype)

    grouped_gemm_cuda(
        A=A,
        B=B,
        C=C,
        output=output,
        M_array=M_array,
        N_array=N_array,
        K_array=K_array,
        is_A_transposed=is_A_transposed,
        is_B_transposed=is_B_transposed,
        alpha=alpha,
        beta=beta,
        benchmark=benchmark,
    )

    return output
