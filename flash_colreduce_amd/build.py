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

OBJ_DIR = os.path.join(HERE, "_build")
PARTS = (0, 1, 2, 3, 4, 5, 6, 7, 8)   # -DFCR_PART=n, see the top of csrc/fcr.hip

HIPCC_FLAGS = [
    "-O3",
    "--offload-arch=gfx950",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    # keep packed fp32 VALU forms out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the scheduler that favours instruction-level parallelism: the masked row sweep gains 3-4 %, the rest is unchanged
    "-mllvm", "-amdgpu-sched-strategy=max-ilp",
]


def hipcc_path() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libfcr.so cannot be built")
    return exe


def build(verbose: bool = True, extra_flags=()) -> str:
    """Compiles the parts of csrc/fcr.hip side by side (one hipcc each) and links them into libfcr.so."""
    hipcc = hipcc_path()
    os.makedirs(OBJ_DIR, exist_ok=True)
    jobs = []
    for part in PARTS:
        obj = os.path.join(OBJ_DIR, f"fcr_part{part}.o")
        # a part uses a subset of the file's helpers
        cmd = [hipcc, *HIPCC_FLAGS, *extra_flags, f"-DFCR_PART={part}", "-Wno-unused-function", "-I", INCLUDE,
               "-c", SRC, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        jobs.append((cmd, obj, subprocess.Popen(cmd)))
    failed = [cmd for cmd, _, proc in jobs if proc.wait() != 0]
    if failed:
        raise subprocess.CalledProcessError(1, failed[0])
    link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *[obj for _, obj, _ in jobs], "-o", LIB]
    if verbose:
        print(" ".join(link), flush=True)
    subprocess.run(link, check=True)
    return LIB


C_CHECK_SRC = os.path.join(ROOT, "tests", "c_abi", "check.c")
C_CHECK_BIN = os.path.join(ROOT, "tests", "c_abi", "check")


def build_c_check(verbose: bool = True) -> str:
    """The plain C caller of the library (tests/c_abi/check.c), linked against libfcr.so next to this file.
    (Compiled as C, where the HIP headers have to be told the platform.)"""
    cmd = [hipcc_path(), "-x", "c", "-O1", "-D__HIP_PLATFORM_AMD__", "-I", INCLUDE, "-I", "/opt/rocm/include", C_CHECK_SRC,
           "-o", C_CHECK_BIN, "-L", HERE, "-lfcr", "-L", "/opt/rocm/lib", "-lamdhip64", "-lm",
           "-Wl,-rpath,$ORIGIN/../../flash_colreduce_amd", "-Wl,-rpath,/opt/rocm/lib"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return C_CHECK_BIN


if __name__ == "__main__":
    build(extra_flags=sys.argv[1:])
    build_c_check()
