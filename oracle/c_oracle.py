"""ctypes wrapper of oracle/_build/liboracle.so (the plain-C restatement of the integer part): TEST INFRASTRUCTURE."""

import ctypes
import os

import numpy as np

from . import build as _build

_lib = None


def _load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_build.LIB):
            _build.build()
        _lib = ctypes.CDLL(_build.LIB)
    return _lib


def continuous_count(x: np.ndarray, size: int) -> np.ndarray:
    x = np.ascontiguousarray(x)
    out = np.empty(size, dtype=np.uint32)
    fn = {np.dtype(np.int32): "oracle_continuous_count_i32", np.dtype(np.int64): "oracle_continuous_count_i64"}[x.dtype]
    getattr(_load(), fn)(
        x.ctypes.data_as(ctypes.c_void_p), ctypes.c_uint64(x.size), ctypes.c_uint32(size),
        out.ctypes.data_as(ctypes.c_void_p),
    )
    return out


def routing_index(ids: np.ndarray, num_experts: int) -> dict[str, np.ndarray]:
    ids = np.ascontiguousarray(ids.reshape(-1), dtype=np.int64)
    R = ids.size
    counts = np.empty(num_experts, np.uint32)
    offsets = np.empty(num_experts, np.uint32)
    cursor = np.empty(num_experts, np.uint32)
    perm, eid, inv = (np.empty(R, np.int32) for _ in range(3))
    p = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    _load().oracle_routing_index(
        p(ids), ctypes.c_int64(R), ctypes.c_uint32(num_experts), p(counts), p(offsets), p(perm), p(eid), p(inv),
        p(cursor),
    )
    return {"counts": counts, "offsets": offsets, "perm": perm, "eid": eid, "inv": inv}
