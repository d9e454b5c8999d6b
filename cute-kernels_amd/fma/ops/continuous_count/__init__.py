"""`continuous_count(x, size)`: how often each of the ids 0 .. size-1 occurs in x, as uint32. The call signature, the
`size == 1` shortcut, the two assertions and the ValueError for an unknown backend are those of the reference's op
(fma/ops/continuous_count/__init__.py:11-43); the counting is `fma_continuous_count` of libfma_hip.so."""

import torch

from ...kernel_backend import KernelBackend, is_hip_kernel_backend
from .cuda_implementation import continuous_count_cuda

_ID_DTYPES = (torch.int32, torch.int64)


@torch.no_grad()
def continuous_count(
    x: torch.Tensor, size: int, *, kernel_backend: KernelBackend = KernelBackend.cuda
) -> torch.Tensor:
    """Histogram of a 1-D tensor of expert ids.

    x: int32 or int64 ids on the GPU. Ids outside [0, size) are skipped (the reference calls this case the caller's
    responsibility). size: number of bins. Returns a uint32 tensor of `size` counts on x's device.
    """
    if size == 1:
        # a single bin takes every element; answered without looking at x, as the reference does (:29-30)
        return torch.tensor([x.numel()], dtype=torch.uint32, device=x.device)

    assert x.dim() == 1, "x should be 1-dimensional"
    assert x.dtype in _ID_DTYPES

    if not is_hip_kernel_backend(kernel_backend):
        raise ValueError(f"unexpected kernel_backend ({kernel_backend})")

    counts = torch.empty(size, dtype=torch.uint32, device=x.device)
    # the launch-shape arguments of the reference's stub are accepted and ignored by the HIP kernel
    continuous_count_cuda(x=x, output=counts, E=size, THREAD_BLOCK_CLUSTER_SIZE=1, BLOCK_SIZE=1024)
    return counts
