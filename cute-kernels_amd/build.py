"""Builds libfma_hip.so (the C-ABI library of HIP kernels for gfx950) in-tree with hipcc.

Usage: python cute-kernels_amd/build.py [--force] [--jobs N]

Each .hip source under csrc/ is compiled to an object file (in parallel) and the objects are linked into
cute-kernels_amd/fma/libfma_hip.so. Without --force a source whose object is newer than it and than every header
is not recompiled.
"""

import argparse
import os
import re
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


# Sources whose kernels count their own outstanding memory operations (s_waitcnt vmcnt(N) with hand-counted N): a
# register spill would add loads and stores of its own and shift those counts, so that LDS stages could be read before
# the operands have landed. Their kernels must use no scratch memory; the build checks the compiler's resource report.
NO_SCRATCH_SOURCES = {"grouped_gemm.hip": "grouped_gemm_kernel", "grouped_gemm_ragged.hip": "ragged_gemm_kernel"}


def _check_no_scratch(src: str, report: str, kernel_substring: str) -> None:
    names = re.findall(r"Function Name: (\S+)", report)
    scratch = re.findall(r"ScratchSize \[bytes/lane\]: (\d+)", report)
    checked = 0
    for name, size in zip(names, scratch):
        if kernel_substring in name:
            checked += 1
            if int(size) != 0:
                raise RuntimeError(f"{src}: kernel {name} uses {size} bytes of scratch per lane (register spills); "
                                   "its hand-counted s_waitcnt values are only valid without scratch traffic")
    if checked == 0:
        raise RuntimeError(f"{src}: the compiler's resource report names no {kernel_substring} kernel")


def _compile_one(src: str, force: bool) -> str:
    obj = os.path.join(OBJ_DIR, os.path.basename(src).replace(".hip", ".o"))
    if not force and os.path.exists(obj):
        newest = max(os.path.getmtime(p) for p in [src] + _headers())
        if os.path.getmtime(obj) >= newest:
            return obj
    guarded = NO_SCRATCH_SOURCES.get(os.path.basename(src))
    cmd = [HIPCC] + FLAGS + (["-Rpass-analysis=kernel-resource-usage"] if guarded else []) + ["-c", src, "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        err = "\n".join(line for line in proc.stderr.splitlines() if "packed-fp32-ops" not in line)
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    stderr = proc.stderr
    if guarded:
        try:
            _check_no_scratch(src, stderr, guarded)
        except RuntimeError:
            os.remove(obj)
            raise
        # the report (remarks with their source excerpts) is not repeated on the console; warnings are
        stderr = "\n".join(line for line in stderr.splitlines() if "warning:" in line)
    # hipcc's host pass warns that it does not know the packed-fp32 feature; that is harmless noise
    err = "\n".join(line for line in stderr.splitlines() if "packed-fp32-ops" not in line)
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
