"""Builds the HIP kernels into ``dice_amd/libdice_moe.so`` for gfx950.

``python -m dice_amd.build`` (or ``build_library()``) cross-compiles without a
GPU.  Objects go to ``dice_amd/_build/``; the shared library stays in-tree next
to this file so it travels with the source tree.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
BUILD_DIR = os.path.join(HERE, "_build")
LIB_PATH = os.path.join(HERE, "libdice_moe.so")

SOURCES = [
    "status.hip",
    "gate.hip",
    "dispatch.hip",
    "combine.hip",
    "modulate.hip",
    "quant.hip",
    "grouped_gemm_f32.hip",
    "grouped_gemm_bf16.hip",
    "grouped_gemm_f16.hip",
    "grouped_gemm_persist.hip",
    "grouped_gemm_persist_f16.hip",
    "grouped_gemm_persist_f8.hip",
    "grouped_mlp.hip",
]

# Packed-fp32 VALU forms are switched off for every device translation unit.
HIP_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-fPIC",
    "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the HIP library cannot be built")
    return exe


def _compile(src: str, extra) -> str:
    obj = os.path.join(BUILD_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *HIP_FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stderr}")
    return obj


def build_library(verbose: bool = True, extra_flags=()) -> str:
    os.makedirs(BUILD_DIR, exist_ok=True)
    jobs = min(len(SOURCES), max(1, min(8, os.cpu_count() or 1)))
    with ThreadPoolExecutor(jobs) as pool:
        objs = list(pool.map(lambda s: _compile(s, list(extra_flags)), SOURCES))
    tmp = LIB_PATH + ".tmp"
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} ({os.path.getsize(LIB_PATH)} bytes)")
    return LIB_PATH


if __name__ == "__main__":
    build_library(extra_flags=sys.argv[1:])
