"""Build-time check of the expert GEMM kernels whose sums live in accumulation
registers that only inline assembly names (csrc/grouped_gemm_persist.hip).

The compiler does not know that those registers are in use.  When it runs out
of vector registers it parks values in accumulation registers of its own
choice, lowest numbers first; a kernel of sixteen blocks owns all 256 and must
see none of that, a kernel of twelve blocks keeps its sums in a64 .. a255 and
leaves a0 .. a63 to the compiler.  A kernel whose k-loop is assembly text
(gemm_persist_kernel4a, gemm_persist_kernel_f8a) also names its register stages, v128 .. v255, in that
text only: it is compiled with a budget of 128 vector registers and must see
the compiler neither above v127 nor in any accumulation register
(gemm_persist_kernel_f8s: the text names v117 .. v127 as well).  This script
reads the device assembly the compiler wrote for a translation unit and fails
the build if an instruction outside the inline assembly touches a register that
belongs to the assembly.
"""
from __future__ import annotations

import re
import sys

_KERNEL = re.compile(r"^(_ZN4dice\S*gemm_persist_kernel(?:4a?|_f8[as])I\S+):")
_ANY_FN = re.compile(r"^(\S+):\s*(;.*)?$")
_REG = re.compile(r"\b([av])(\d+)\b|\b([av])\[(\d+):(\d+)\]")


def _owned_from(mangled: str):
    """(first accumulation register, first vector register) the assembly owns."""
    if "gemm_persist_kernel4aI" in mangled or "gemm_persist_kernel_f8aI" in mangled:
        return 0, 128
    if "gemm_persist_kernel_f8sI" in mangled:     # the scaled kind's text also names v117 .. v127
        return 0, 117
    # gemm_persist_kernel4<MODE, HAS_BIAS, BN, ...>: ILi<mode>ELb<bias>ELi<BN>E...
    m = re.search(r"gemm_persist_kernel4ILi\d+ELb[01]ELi(\d+)E", mangled)
    if not m:
        raise RuntimeError(f"cannot read the tile width from {mangled}")
    return (0 if int(m.group(1)) == 256 else 64), 256


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
            first_acc, first_vec = _owned_from(kernel)
            for m in _REG.finditer(code):
                if m.group(1):
                    file_, regs = m.group(1), [int(m.group(2))]
                else:
                    file_, regs = m.group(3), range(int(m.group(4)), int(m.group(5)) + 1)
                if any(r >= (first_acc if file_ == "a" else first_vec) for r in regs):
                    problems.append(f"{kernel}: {code.strip()}")
    if problems:
        raise RuntimeError(
            "the compiler placed values of its own in registers that belong to the kernel's assembly "
            f"({len(problems)} instructions), e.g.\n  " + "\n  ".join(problems[:8]))
    if not checked:
        raise RuntimeError(f"{asm_path}: no checked kernel found")
    return len(checked)


if __name__ == "__main__":
    for path in sys.argv[1:]:
        print(f"{path}: {check(path)} kernels, the assembly's registers untouched by the compiler")
