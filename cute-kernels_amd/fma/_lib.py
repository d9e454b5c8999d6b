"""ctypes binding of libfma_hip.so, the C-ABI library of HIP kernels (declared in include/fma_hip.h).

This is the replacement of the reference's `cpp_jit` boundary (fma/jit.py:90-159): instead of JIT-compiling
pybind11 extensions on first call, one pre-built shared library is loaded once and called with raw device
pointers, sizes and the current HIP stream. There is no fallback: if the library is missing, or a call fails,
a RuntimeError is raised.
"""

import ctypes
import os
import threading

import torch


_LIB_NAME = "libfma_hip.so"
# FMA_HIP_LIBRARY names another build of the same library (e.g. one compiled with different tuning macros)
_LIB_PATH = os.environ.get("FMA_HIP_LIBRARY") or os.path.join(os.path.dirname(os.path.abspath(__file__)), _LIB_NAME)
_ABI_VERSION = 2

FMA_F32, FMA_F16, FMA_BF16 = 0, 1, 2
FMA_VARY_M, FMA_VARY_K = 0, 1
_DTYPE_CODE = {torch.float32: FMA_F32, torch.float16: FMA_F16, torch.bfloat16: FMA_BF16}

_p = ctypes.c_void_p
_i64 = ctypes.c_int64
_i32 = ctypes.c_int
_f32 = ctypes.c_float

# name -> (restype, argtypes); one entry per declaration of include/fma_hip.h
SIGNATURES = {
    "fma_last_error_string": (ctypes.c_char_p, []),
    "fma_abi_version": (_i32, []),
    "fma_num_compute_units": (_i32, []),
    "fma_continuous_count_workspace_bytes": (_i64, [_i64, _i64]),
    "fma_continuous_count": (_i32, [_p, _i32, _i64, _p, _i64, _p, _i64, _p]),
    "fma_moe_build_index_workspace_bytes": (_i64, [_i64, _i64]),
    "fma_moe_build_index": (_i32, [_p, _i32, _i64, _i64, _p, _p, _p, _p, _p, _p, _i64, _p]),
    "fma_moe_build_index_static_max_words": (_i64, []),
    "fma_moe_build_index_static": (_i32, [_p, _i32, _i64, _i64, _p, _p, _p, _p, _p, _p]),
    "fma_gather_rows": (_i32, [_p, _p, _i64, _i64, _i32, _p, _i32, _p]),
    "fma_dispatch_rows": (_i32, [_p, _p, _i64, _i64, _i64, _p, _i32, _p]),
    "fma_combine": (_i32, [_p, _p, _p, _i64, _i64, _i64, _p, _i32, _p]),
    "fma_combine_bwd": (_i32, [_p, _p, _p, _p, _i64, _i64, _i64, _p, _p, _i32, _p]),
    "fma_swiglu_forward": (_i32, [_p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i32, _p]),
    "fma_swiglu_backward": (_i32, [_p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _p]),
    "fma_grouped_gemm": (_i32, [_p, _p, _p, _p, _p, _p, _i64, _i32, _i32, _f32, _i32, _p]),
    "fma_grouped_gemm_ragged": (_i32, [_p, _p, _p, _p, _p, _i64, _i32, _i64, _i64, _i64, _i32, _i32, _f32, _i32, _p]),
    "fma_grouped_gemm_swiglu_bwd": (_i32, [_p, _p, _p, _p, _p, _i64, _i64, _i64, _i32, _p]),
    "fma_grouped_gemm_gathered": (_i32, [_p, _i64, _p, _i32, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i32, _i32, _p]),
    "fma_grouped_gemm_gathered_wgrad": (_i32, [_p, _p, _i64, _p, _i32, _p, _p, _i64, _i64, _i64, _f32, _i32, _p]),
    "fma_grouped_gemm_swiglu": (_i32, [_p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i32, _p]),
    "fma_expert_bias_add": (_i32, [_p, _p, _p, _i64, _i64, _i64, _i32, _p]),
    "fma_expert_bias_grad_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "fma_expert_bias_grad": (_i32, [_p, _p, _i64, _i64, _i64, _p, _p, _i64, _i32, _p]),
    "fma_router_topk": (_i32, [_p, _p, _i64, _i64, _i64, _i64, _p, _p, _p, _p, _p, _i32, _p]),
    "fma_moe_build_index_from_hist": (_i32, [_p, _i64, _i64, _i64, _p, _p, _p, _p, _p, _p, _p]),
    "fma_router_topk_bwd": (_i32, [_p, _p, _p, _p, _i64, _i64, _i64, _p, _i32, _p]),
    "fma_fused_residual_add_rmsnorm_fwd": (_i32, [_p, _p, _p, _p, _p, _p, _i64, _i64, _f32, _f32, _i32, _p]),
    "fma_fused_residual_add_rmsnorm_bwd_workspace_bytes": (_i64, [_i64, _i64]),
    "fma_fused_residual_add_rmsnorm_bwd": (
        _i32, [_p, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _f32, _f32, _p, _i64, _i32, _p],
    ),
}

_lib = None
_lock = threading.Lock()


def library_path() -> str:
    return _LIB_PATH


def load() -> ctypes.CDLL:
    """Loads the library once and types every entry point. Raises RuntimeError if it was not built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                f"{_LIB_PATH} is missing: build it with `python cute-kernels_amd/build.py` "
                "(there is no non-HIP implementation of these ops)"
            )
        lib = ctypes.CDLL(_LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        version = lib.fma_abi_version()
        if version != _ABI_VERSION:
            raise RuntimeError(f"{_LIB_NAME} has ABI version {version}, this package expects {_ABI_VERSION}")
        _lib = lib
    return _lib


def check(rc: int, what: str) -> None:
    """Turns a non-zero return code of an entry point into the RuntimeError the reference's TORCH_CHECKs raise."""
    if rc != 0:
        message = load().fma_last_error_string().decode("utf-8", "replace")
        raise RuntimeError(f"{what} failed with code {rc}: {message}")


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {dtype}") from None


def ptr(tensor: torch.Tensor | None) -> int | None:
    return None if tensor is None else tensor.data_ptr()


def require_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("this op runs on the GPU only: got a tensor on " + str(t.device))


def current_stream(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream
