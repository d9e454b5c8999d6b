"""`continuous_count`: histogram of expert ids. Mirrors fma/ops/continuous_count/__init__.py:11-43 of the reference."""

import torch

from ...kernel_backend import KernelBackend, is_hip_kernel_backend
from .cuda_implementation import continuous_count_cuda


@torch.no_grad()
def continuous_count(
    x: torch.Tensor, size: int, *, kernel_backend: KernelBackend = KernelBackend.cuda
) -> torch.Tensor:
    """counts the number of occurances of the values [0, 1, ..., `size`) in the input tensor (`size` is excluded).
        NOTE: values outside this range are ignored and not counted.

    Args:
        x (torch.Tensor): 1-dimensional int32 or int64 tensor on the GPU
        size (int): values [0, 1, ..., `size`) are counted (`size` is excluded)
        kernel_backend (KernelBackend, optional): KernelBackend.cuda (the HIP kernel). Defaults to KernelBackend.cuda.

    Returns:
        torch.Tensor: uint32 tensor of `size` counts
    """

    if size == 1:
        return torch.tensor([x.numel()], dtype=torch.uint32, device=x.device)

    assert x.dim() == 1, "x should be 1-dimensional"
    assert x.dtype in [torch.int32, torch.long]

    if is_hip_kernel_backend(kernel_backend):
        output = torch.empty(size, dtype=torch.uint32, device=x.device)
        continuous_count_cuda(x=x, output=output, E=size, THREAD_BLOCK_CLUSTER_SIZE=1, BLOCK_SIZE=1024)
    else:
        raise ValueError(f"unexpected kernel_backend ({kernel_backend})")

    return output
