"""Builds libffi_hip.so (the C-ABI library with the gfx950 kernels) in-tree with hipcc.

Usage: ``python ecml23-sparse_amd/build.py [--force]``.  The same steps are available through
CMake (``csrc/CMakeLists.txt``); this script exists so that the build needs nothing but hipcc.
"""
from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
OBJ_DIR = os.path.join(HERE, "build")
LIB_PATH = os.path.join(HERE, "libffi_hip.so")

SOURCES = [
    "ffi_api.hip",
    "ffi_forward.hip",
    "ffi_weight_grad.hip",
    "ffi_input_grad.hip",
    "ffi_plan.hip",
    "ffi_util.hip",
    "ffi_wide.hip",
    "ffi_bf16.hip",
    "ffi_loss.hip",
    "ffi_sparse_grad.hip",
    "ffi_optimizer.hip",
    "ffi_rewire.hip",
    "ffi_fallback.hip",
    "host/ffi_host_kernels.cc",
]

# gfx950 only.  Packed-fp32 VALU forms are switched off for all device code.
HIPCC_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
    "-I", INCLUDE, "-I", CSRC,
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the HIP kernels cannot be built")
    return exe


def _compile(src: str) -> str:
    obj = os.path.join(OBJ_DIR, os.path.splitext(os.path.basename(src))[0] + ".o")
    cmd = [hipcc(), *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{proc.stdout}\n{proc.stderr}")
    return obj


def build(force: bool = True, jobs: int | None = None) -> str:
    """Compiles every HIP source and links the shared library; returns its path."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    if force and os.path.exists(LIB_PATH):
        os.remove(LIB_PATH)
    jobs = jobs or min(len(SOURCES), max(1, (os.cpu_count() or 2) // 2))
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(_compile, SOURCES))
    cmd = [hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB_PATH, *objs]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
    return LIB_PATH


if __name__ == "__main__":
    print(build(force="--force" in sys.argv or True))
