"""CPU checks of the C-ABI boundary: the library loads without a GPU, exports every symbol include/fma_hip.h declares,
and rejects bad arguments with an error code and a message before anything is launched."""

import ctypes
import os
import re

import pytest

from fma import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols() -> list[str]:
    text = open(os.path.join(ROOT, "include", "fma_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fma_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    declared = _declared_symbols()
    assert declared, "no declarations parsed from include/fma_hip.h"
    assert declared == sorted(_lib.SIGNATURES), "ctypes signatures and the header list different entry points"


def test_library_exports_every_declared_symbol(lib):
    for name in _declared_symbols():
        assert hasattr(lib, name), f"libfma_hip.so does not export {name}"
    assert lib.fma_abi_version() == 2


def test_workspace_queries(lib):
    assert lib.fma_continuous_count_workspace_bytes(16 << 20, 64) >= 256 + 64 * 4
    assert lib.fma_moe_build_index_workspace_bytes(1024, 8) == 2 * 8 * 4  # two 512-slot chunks
    assert lib.fma_moe_build_index_workspace_bytes(0, 8) == 8 * 4


def _err(lib) -> str:
    return lib.fma_last_error_string().decode()


def test_continuous_count_validation(lib):
    buf = ctypes.create_string_buffer(4096 + 16)
    p = (ctypes.addressof(buf) + 15) & ~15  # a 16-byte aligned, non-NULL (host) address: never dereferenced
    assert lib.fma_continuous_count(p, 2, 10, p, 64, p, 4096, None) == -2 and "int32 or int64" in _err(lib)
    assert lib.fma_continuous_count(p, 4, 10, p, 0, p, 4096, None) == -3
    assert lib.fma_continuous_count(p, 4, 10, p, 16385, p, 4096, None) == -4 and "16384" in _err(lib)  # E limit
    assert lib.fma_continuous_count(p, 4, 1 << 32, p, 64, p, 4096, None) == -5  # n limit 2^32-1
    assert lib.fma_continuous_count(p, 4, 10, None, 64, p, 4096, None) == -1
    assert lib.fma_continuous_count(p + 4, 4, 10, p, 64, p, 4096, None) == -6 and "aligned" in _err(lib)
    assert lib.fma_continuous_count(p, 4, 10, p, 64, p, 16, None) == -7 and "workspace" in _err(lib)


def test_build_index_validation(lib):
    buf = ctypes.create_string_buffer(4096 + 16)
    p = (ctypes.addressof(buf) + 15) & ~15
    assert lib.fma_moe_build_index(p, 4, 10, 1025, p, p, p, p, p, p, 1 << 20, None) == -4  # E limit 1024
    assert lib.fma_moe_build_index(p, 4, 10, 8, p, p, None, p, p, p, 1 << 20, None) == -1
    assert lib.fma_moe_build_index(p, 4, 1 << 31, 8, p, p, p, p, p, p, 1 << 40, None) == -5
    assert lib.fma_moe_build_index(p, 4, 10_000, 8, p, p, p, p, p, p, 8, None) == -7


def test_row_kernels_validation(lib):
    buf = ctypes.create_string_buffer(4096 + 16)
    p = (ctypes.addressof(buf) + 15) & ~15
    assert lib.fma_gather_rows(p, p, 4, 0, 1, p, 2, None) == -3 and "row length" in _err(lib)  # any H >= 1 is served
    assert lib.fma_gather_rows(p, p, 4, 16, 0, p, 2, None) == -3  # divisor < 1
    assert lib.fma_gather_rows(p, p, 4, 16, 1, p, 7, None) == -2  # dtype code
    assert lib.fma_dispatch_rows(p, p, 4, 0, 16, p, 2, None) == -3  # top_k < 1
    assert lib.fma_dispatch_rows(p, None, 4, 2, 16, p, 2, None) == -1
    assert lib.fma_dispatch_rows(p, p, 0, 2, 16, p, 2, None) == 0
    assert lib.fma_combine(p, p, p, 4, 0, 16, p, 2, None) == -3  # top_k < 1
    assert lib.fma_combine(p + 1, p, p, 4, 2, 16, p, 2, None) == -6  # not even aligned to the element size
    assert lib.fma_combine_bwd(p, None, p, p, 4, 2, 16, p, p, 2, None) == -1  # d_gates needs o
    assert lib.fma_gather_rows(p, p, 0, 16, 1, p, 2, None) == 0  # empty input: nothing to do
    assert lib.fma_combine(p, p, p, 0, 2, 16, p, 2, None) == 0


def test_swiglu_and_gemm_validation(lib):
    buf = ctypes.create_string_buffer(4096 + 16)
    p = (ctypes.addressof(buf) + 15) & ~15
    assert lib.fma_swiglu_forward(p, p, p, 4, 8, 4, 8, 8, 2, None) == -3 and "stride" in _err(lib)
    assert lib.fma_swiglu_forward(p, p, p, 4, 8, 8, 8, 8, 9, None) == -2
    assert lib.fma_swiglu_forward(p, p, p, 0, 8, 8, 8, 8, 2, None) == 0
    assert lib.fma_swiglu_backward(p, p, p, p, None, 4, 8, 8, 8, 8, 8, 8, 2, None) == -1
    assert lib.fma_grouped_gemm(p, p, p, p, p, p, 1025, 0, 1, 1.0, 2, None) == -4 and "1024" in _err(lib)
    assert lib.fma_grouped_gemm(p + 4, p, p, p, p, p, 4, 0, 1, 1.0, 0, None) == -6  # fp32 operands: same alignment rule
    assert lib.fma_grouped_gemm_swiglu(p, p, None, p, p, p, 4, 16, 64, 0, None) == -8  # the fused epilogue is 16-bit only
    assert lib.fma_grouped_gemm(p, p, p, p, p, p, 4, 0, 1, 1.0, 5, None) == -2
    assert lib.fma_grouped_gemm(p, p, p, None, p, p, 4, 0, 1, 1.0, 2, None) == -1
    assert lib.fma_grouped_gemm(p, p, p, p, p, p, 0, 0, 1, 1.0, 2, None) == 0
    assert lib.fma_grouped_gemm_swiglu(p, p, None, p, p, p, 4, 12, 64, 2, None) == -3  # I % 8 != 0
    assert lib.fma_grouped_gemm_swiglu(p, p, None, p, p, p, 4, 16, 60, 2, None) == -3  # K % 8 != 0
    assert lib.fma_grouped_gemm_swiglu(p, p, None, p, p, p, 4, 1 << 22, 64, 2, None) == -3  # beyond the 32-bit tile offsets
    assert lib.fma_grouped_gemm_swiglu(p, p, None, p, p, p, 4, 16, 1 << 21, 2, None) == -3


def test_router_norm_and_bias_validation(lib):
    buf = ctypes.create_string_buffer(4096 + 16)
    p = (ctypes.addressof(buf) + 15) & ~15
    # router: T, H, E, top_k
    assert lib.fma_router_topk(p, p, 4, 64, 8, 9, p, p, p, None, None, 2, None) == -3 and "top_k" in _err(lib)
    assert lib.fma_router_topk(p, p, 4, 64, 8, 65, p, p, p, None, None, 2, None) == -3
    assert lib.fma_router_topk(p, p, 4, 60, 8, 2, p, p, p, None, None, 2, None) == -3 and "multiple of 8" in _err(lib)
    assert lib.fma_router_topk(p, p, 4, 64, 1025, 2, p, p, p, None, None, 2, None) == -4
    assert lib.fma_router_topk(p, p, 4, 64, 8, 2, p, p, p, None, None, 0, None) == -2  # 16-bit dtypes only
    assert lib.fma_router_topk(p, p, 4, 64, 8, 2, None, p, p, None, None, 2, None) == -1
    assert lib.fma_router_topk(p + 2, p, 4, 64, 8, 2, p, p, p, None, None, 2, None) == -6
    assert lib.fma_router_topk(p, p, 0, 64, 8, 2, p, p, p, None, None, 2, None) == 0
    assert lib.fma_router_topk_bwd(p, p, None, None, 4, 8, 9, p, 2, None) == -3
    assert lib.fma_router_topk_bwd(p, None, None, None, 4, 8, 2, p, 2, None) == -1
    # residual add + RMSNorm: B, H
    assert lib.fma_fused_residual_add_rmsnorm_fwd(p, p, None, p, p, None, 4, 0, 1e-5, 1.0, 0, None) == -3
    assert lib.fma_fused_residual_add_rmsnorm_fwd(p, p, None, p, p, None, 4, 65537, 1e-5, 1.0, 0, None) == -3
    assert lib.fma_fused_residual_add_rmsnorm_fwd(p, p, None, p, p, None, 4, 64, 1e-5, 1.0, 3, None) == -2
    assert lib.fma_fused_residual_add_rmsnorm_fwd(p, None, None, p, p, None, 4, 64, 1e-5, 1.0, 0, None) == -1
    assert lib.fma_fused_residual_add_rmsnorm_fwd(p, p, None, p, p, None, 0, 64, 1e-5, 1.0, 0, None) == 0
    assert lib.fma_fused_residual_add_rmsnorm_bwd_workspace_bytes(16384, 4096) % (4096 * 4) == 0
    assert lib.fma_fused_residual_add_rmsnorm_bwd_workspace_bytes(0, 4096) == 0
    # weight without weight_grad
    assert lib.fma_fused_residual_add_rmsnorm_bwd(p, p, p, None, None, p, p, None, 4, 64, 1e-5, 1.0, p, 4096, 0, None) == -1
    # expert bias: E, R, N
    assert lib.fma_expert_bias_add(p, p, p, 2, 4, 12, 2, None) == -3 and "16 bytes" in _err(lib)
    assert lib.fma_expert_bias_add(p, p, p, 1025, 4, 16, 2, None) == -4
    assert lib.fma_expert_bias_add(p, None, p, 2, 4, 16, 2, None) == -1
    assert lib.fma_expert_bias_add(p, p, p, 2, 0, 16, 2, None) == 0
    assert lib.fma_expert_bias_grad_workspace_bytes(8, 32768, 4096) == (32768 // 256 + 8) * 4096 * 4
    assert lib.fma_expert_bias_grad(p, p, 2, 1000, 16, p, p, 8, 2, None) == -7 and "workspace" in _err(lib)


def test_check_raises_runtime_error(lib):
    rc = lib.fma_continuous_count(None, 4, 10, None, 64, None, 0, None)
    with pytest.raises(RuntimeError, match="counts is NULL"):
        _lib.check(rc, "continuous_count_cuda")
