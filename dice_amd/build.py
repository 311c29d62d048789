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


# Translation units whose kernels keep their sums in accumulation registers that
# the compiler does not know about: their device assembly is kept and checked
# (check_acc_regs.py) before the library is linked.
ACC_CHECKED = {"grouped_gemm_persist.hip", "grouped_gemm_persist_f16.hip", "grouped_gemm_persist_f8.hip"}


def _generate_sources() -> None:
    """Writes the generated k-loop of the expert GEMM (csrc/gen_persist64_asm.py) into the
    build directory, which is on the include path of every translation unit."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("gen_persist64_asm", os.path.join(CSRC, "gen_persist64_asm.py"))
    gen = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(gen)
    text = gen.generate()
    path = os.path.join(BUILD_DIR, "persist64_asm.inc")
    if not os.path.exists(path) or open(path).read() != text:
        with open(path, "w") as f:
            f.write(text)


def _compile(src: str, extra) -> str:
    stem = os.path.splitext(src)[0]
    obj = os.path.join(BUILD_DIR, stem + ".o")
    cmd = [_hipcc(), *HIP_FLAGS, "-I", BUILD_DIR, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    if src in ACC_CHECKED:
        cmd.insert(-4, "-save-temps=obj")
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stderr}")
    if src in ACC_CHECKED:
        from dice_amd.check_acc_regs import check
        check(os.path.join(BUILD_DIR, stem + "-hip-amdgcn-amd-amdhsa-gfx950.s"))
    return obj


def build_library(verbose: bool = True, extra_flags=(), out: str = None) -> str:
    """Compiles every source and links the library (to ``out`` instead of the
    package's own path when given: a second build to compare with, e.g.
    ``python -m dice_amd.build --out /tmp/other.so -DDICE_MFMA_ROWS_OUTERMOST=1``)."""
    target = os.path.abspath(out) if out else LIB_PATH
    os.makedirs(BUILD_DIR, exist_ok=True)
    _generate_sources()
    jobs = min(len(SOURCES), max(1, min(8, os.cpu_count() or 1)))
    with ThreadPoolExecutor(jobs) as pool:
        objs = list(pool.map(lambda s: _compile(s, list(extra_flags)), SOURCES))
    tmp = target + ".tmp"
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    os.replace(tmp, target)
    if verbose:
        print(f"built {target} ({os.path.getsize(target)} bytes)")
    return target


if __name__ == "__main__":
    argv = sys.argv[1:]
    out_path = None
    if "--out" in argv:
        at = argv.index("--out")
        out_path = argv[at + 1]
        del argv[at:at + 2]
    build_library(extra_flags=argv, out=out_path)
