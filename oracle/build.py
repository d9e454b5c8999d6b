"""Builds the C part of the CPU oracle (oracle/count_index.c) into oracle/_build/liboracle.so with gcc.

The reference itself has nothing that compiles here: its native sources are CUDA (nvcc, cooperative-groups clusters)
and CUTLASS (an empty submodule), so there is no oracle/_ref build.
"""

import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
OUT_DIR = os.path.join(HERE, "_build")
LIB = os.path.join(OUT_DIR, "liboracle.so")


def build() -> str:
    os.makedirs(OUT_DIR, exist_ok=True)
    subprocess.run(
        ["gcc", "-O2", "-shared", "-fPIC", os.path.join(HERE, "count_index.c"), "-o", LIB], check=True
    )
    return LIB


if __name__ == "__main__":
    print(build())
