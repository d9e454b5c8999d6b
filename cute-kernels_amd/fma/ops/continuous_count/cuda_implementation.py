"""`continuous_count_cuda` custom op: same name, arguments and mutation contract as the reference's stub
(fma/ops/continuous_count/cuda_implementation/__init__.py:12-16), bound to fma_continuous_count of libfma_hip.so."""

import torch
from torch.library import custom_op

from ... import _lib
from ...constants import LIBRARY_NAME


@custom_op(f"{LIBRARY_NAME}::continuous_count_cuda", mutates_args={"output"})
def continuous_count_cuda(
    x: torch.Tensor, output: torch.Tensor, E: int, THREAD_BLOCK_CLUSTER_SIZE: int, BLOCK_SIZE: int
) -> None:
    # THREAD_BLOCK_CLUSTER_SIZE and BLOCK_SIZE are launch-shape hints of the CUDA kernel; the wave64 kernel
    # chooses its own launch shape
    _lib.require_gpu(x, output)
    assert output.dtype == torch.uint32 and output.numel() == E and output.is_contiguous()
    assert x.dtype in (torch.int32, torch.int64)
    x = x.contiguous()
    lib = _lib.load()
    n = x.numel()
    with torch.cuda.device(x.device):
        # per-workgroup partial histograms; uninitialised memory from the caching allocator, owned by this call
        ws = torch.empty(max(lib.fma_continuous_count_workspace_bytes(n, E), 4), dtype=torch.uint8, device=x.device)
        rc = lib.fma_continuous_count(
            x.data_ptr(), x.element_size(), n, output.data_ptr(), E, ws.data_ptr(), ws.numel(),
            _lib.current_stream(x.device),
        )
    _lib.check(rc, "continuous_count_cuda")
