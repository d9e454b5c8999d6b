"""Kernel backend selector, kept for call-signature compatibility with the reference (fma/kernel_backend.py:11-14).

`cuda` selects the HIP kernels (the device type of PyTorch-ROCm is "cuda"). `triton` is accepted and served by the
same HIP kernels, because the reference's MoE and swiglu_packed default to it and there is no Triton code here.
`torch` names the reference's own eager implementation; it is not part of this package and every op raises
ValueError for it, exactly as for any other unexpected value.
"""

from enum import Enum


class KernelBackend(Enum):
    cuda = "cuda"
    torch = "torch"
    triton = "triton"


def is_hip_kernel_backend(kernel_backend: KernelBackend) -> bool:
    return kernel_backend in (KernelBackend.cuda, KernelBackend.triton)
