"""Builds libfma_hip.so (the C-ABI library of HIP kernels for gfx950) in-tree with hipcc.

Usage: python cute-kernels_amd/build.py [--force] [--jobs N]

Each .hip source under csrc/ is compiled to an object file (in parallel) and the objects are linked into
cute-kernels_amd/fma/libfma_hip.so. Without --force a source whose object is newer than it and than every header
is not recompiled.
"""

import argparse
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB_PATH = os.path.join(HERE, "fma", "libfma_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -packed-fp32-ops is switched off: the packed fp32 forms have produced silently wrong results on this hardware pool
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-I" + os.path.join(REPO, "include"),
    "-I" + CSRC,
]


def _sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _headers() -> list[str]:
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    headers.append(os.path.join(REPO, "include", "fma_hip.h"))
    return headers


def _compile_one(src: str, force: bool) -> str:
    obj = os.path.join(OBJ_DIR, os.path.basename(src).replace(".hip", ".o"))
    if not force and os.path.exists(obj):
        newest = max(os.path.getmtime(p) for p in [src] + _headers())
        if os.path.getmtime(obj) >= newest:
            return obj
    cmd = [HIPCC] + FLAGS + ["-c", src, "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass warns that it does not know the packed-fp32 feature; that is harmless noise
    err = "\n".join(line for line in proc.stderr.splitlines() if "packed-fp32-ops" not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(force: bool = False, jobs: int = 4) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        objs = list(pool.map(lambda s: _compile_one(s, force), _sources()))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    return LIB_PATH


if __name__ == "__main__":
    parser = argparse.ArgumentParser()
    parser.add_argument("--force", action="store_true")
    parser.add_argument("--jobs", type=int, default=4)
    ns = parser.parse_args()
    print(build(force=ns.force, jobs=ns.jobs))
