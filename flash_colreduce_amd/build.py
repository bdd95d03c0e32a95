"""Builds libfcr.so (the C-ABI HIP library) in-tree for gfx950.

    python -m flash_colreduce_amd.build

hipcc cross-compiles without a GPU, so this runs anywhere the ROCm toolchain is installed.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SRC = os.path.join(HERE, "csrc", "fcr.hip")
INCLUDE = os.path.join(ROOT, "include")
LIB = os.path.join(HERE, "libfcr.so")

HIPCC_FLAGS = [
    "-O3",
    "--offload-arch=gfx950",
    "-std=c++17",
    "-shared",
    "-fPIC",
    "-fno-gpu-rdc",
    # keep packed fp32 VALU forms out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc_path() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libfcr.so cannot be built")
    return exe


def build(verbose: bool = True, extra_flags=()) -> str:
    cmd = [hipcc_path(), *HIPCC_FLAGS, *extra_flags, "-I", INCLUDE, SRC, "-o", LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    build(extra_flags=sys.argv[1:])
