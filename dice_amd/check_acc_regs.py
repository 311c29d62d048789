"""Build-time check of the expert GEMM kernels whose sums live in accumulation
registers that only inline assembly names (csrc/grouped_gemm_persist.hip).

The compiler does not know that those registers are in use.  When it runs out
of vector registers it parks values in accumulation registers of its own
choice, lowest numbers first; a kernel of sixteen blocks owns all 256 and must
see none of that, a kernel of twelve blocks keeps its sums in a64 .. a255 and
leaves a0 .. a63 to the compiler.  This script reads the device assembly the
compiler wrote for a translation unit and fails the build if an instruction
outside the inline assembly touches a register the kernel's sums occupy.
"""
from __future__ import annotations

import re
import sys

_KERNEL = re.compile(r"^(_ZN4dice\S*gemm_persist_kernel4I\S+):")
_ANY_FN = re.compile(r"^(\S+):\s*(;.*)?$")
_REG = re.compile(r"\ba(\d+)\b|\ba\[(\d+):(\d+)\]")


def _tile_width(mangled: str) -> int:
    # gemm_persist_kernel4<MODE, HAS_BIAS, BN, ...>: ILi<mode>ELb<bias>ELi<BN>E...
    m = re.search(r"gemm_persist_kernel4ILi\d+ELb[01]ELi(\d+)E", mangled)
    if not m:
        raise RuntimeError(f"cannot read the tile width from {mangled}")
    return int(m.group(1))


def check(asm_path: str) -> int:
    """Returns the number of checked kernels; raises on a collision."""
    kernel = None
    in_asm = False
    checked = set()
    problems = []
    with open(asm_path) as f:
        for line in f:
            m = _KERNEL.match(line)
            if m:
                kernel = m.group(1)
                checked.add(kernel)
                continue
            if line.startswith("_Z") and _ANY_FN.match(line):
                kernel = None
                continue
            if ";;#ASMSTART" in line:
                in_asm = True
                continue
            if ";;#ASMEND" in line:
                in_asm = False
                continue
            if in_asm or kernel is None or line.startswith("\t."):
                continue
            code = line.split(";")[0]
            first_owned = 0 if _tile_width(kernel) == 256 else 64
            for m in _REG.finditer(code):
                regs = [int(m.group(1))] if m.group(1) else range(int(m.group(2)), int(m.group(3)) + 1)
                if any(r >= first_owned for r in regs):
                    problems.append(f"{kernel}: {code.strip()}")
    if problems:
        raise RuntimeError(
            "the compiler placed values of its own in accumulation registers that hold the kernel's sums "
            f"({len(problems)} instructions), e.g.\n  " + "\n  ".join(problems[:8]))
    if not checked:
        raise RuntimeError(f"{asm_path}: no gemm_persist_kernel4 instantiation found")
    return len(checked)


if __name__ == "__main__":
    for path in sys.argv[1:]:
        print(f"{path}: {check(path)} kernels, accumulation registers untouched by the compiler")
