"""The generated k-loop of the expert GEMM (dice_amd/csrc/gen_persist64_asm.py): what the
generator must guarantee whatever its schedule, checked on the text it writes (no GPU).

An independent replay of every statement sequence the kernel runs (prologue, then tiles of
steps) with in-order LDS and vector-memory queues: every MFMA reads fragments whose LDS reads
have completed under the waits in the text, every LDS write sends a stage register whose load
has completed, no load refills a stage register before the LDS write that reads it was issued,
and every register stays inside the plan the build-time checker assumes.
"""
import importlib.util
import os
import re

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
GEN = os.path.join(HERE, "..", "dice_amd", "csrc", "gen_persist64_asm.py")


def _load():
    spec = importlib.util.spec_from_file_location("gen_persist64_asm", GEN)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _regs(tok):
    m = re.fullmatch(r"([av])\[(\d+):(\d+)\]", tok)
    assert m, tok
    return m.group(1), int(m.group(2)), int(m.group(3))


class Replay:
    """In-order queues; `done` counts completed operations of each queue."""

    def __init__(self):
        self.lds_issued = self.lds_done = 0
        self.vm_issued = self.vm_done = 0
        self.frag_ready = {}      # first register of a fragment -> index of the LDS read filling it
        self.stage_ready = {}     # first register of a stage entry -> index of the load filling it
        self.stage_sent = {}      # first register of a stage entry -> True once its LDS write was issued
        self.mfma = 0

    def run(self, lines):
        for ln in lines:
            op, _, rest = ln.partition(" ")
            args = [a.strip() for a in rest.split(",")]
            if op == "s_waitcnt":
                m = re.fullmatch(r"(lgkmcnt|vmcnt)\((\d+)\)", rest.strip())
                assert m, ln
                if m.group(1) == "lgkmcnt":
                    self.lds_done = max(self.lds_done, self.lds_issued - int(m.group(2)))
                else:
                    self.vm_done = max(self.vm_done, self.vm_issued - int(m.group(2)))
            elif op == "s_barrier":
                assert self.lds_done == self.lds_issued, "barrier with LDS operations in flight"
            elif op == "MFMA":
                (fa, a0, a1), (_, w0, w1), (_, r0, r1) = _regs(args[0]), _regs(args[1]), _regs(args[2])
                assert fa == "a" and a1 - a0 == 15 and a0 % 16 == 0 and a1 < 256
                assert w1 - w0 == 3 and r1 - r0 == 3 and w1 < 64 and r1 < 64
                assert args[3] in ("0", args[0])
                for f in (w0, r0):
                    assert f in self.frag_ready, f"fragment v{f} never read"
                    assert self.frag_ready[f] < self.lds_done, f"{ln}: fragment v{f} still in flight"
                self.mfma += 1
            elif op == "ds_read_b128":
                _, d0, d1 = _regs(args[0])
                assert d1 - d0 == 3 and d1 < 64
                self.frag_ready[d0] = self.lds_issued
                self.lds_issued += 1
            elif op == "ds_write_b128":
                _, d0, d1 = _regs(args[1].split(" ")[0])
                assert d1 - d0 == 3 and 128 <= d0 and d1 < 256
                assert d0 in self.stage_ready and self.stage_ready[d0] < self.vm_done, f"{ln}: load in flight"
                self.stage_sent[d0] = True
                self.lds_issued += 1
            elif op == "buffer_load_dwordx4":
                _, d0, d1 = _regs(args[0])
                assert d1 - d0 == 3 and 128 <= d0 and d1 < 256
                # (an LDS write reads its data register when it issues: in-order issue is enough)
                assert self.stage_sent.get(d0, True), f"{ln}: refilled before it was sent to LDS"
                self.stage_ready[d0] = self.vm_issued
                self.stage_sent[d0] = False
                self.vm_issued += 1
            else:
                raise AssertionError(f"unexpected instruction {ln}")


@pytest.mark.parametrize("kind", [0, 1])
@pytest.mark.parametrize("live", [1, 2, 3, 4])
def test_generated_loop_waits_cover_every_dependence(kind, live):
    gen = _load()
    pcs = gen.simulate(kind, live)
    tn = gen.KINDS[kind]["TN"]
    assert sorted(pcs) == ["abc_s0_v0", "abc_s0_v1", "abc_s1_v0", "d_s0", "d_s1", "load_q0_stage1",
                           "load_step0", "load_step1", "read_first", "write_q0_stage1", "write_step0"]
    r = Replay()
    for name in ("load_step0", "load_step1", "write_step0", "load_step0", "write_q0_stage1", "load_q0_stage1"):
        r.run(pcs[name])
    r.lds_done = r.lds_issued                      # s_waitcnt lgkmcnt(0) + barrier in the kernel's own code
    for tile_steps in (6, 18, 8):                  # (even step counts of at least six, as the launcher admits)
        r.run(pcs["read_first"])
        before = r.mfma
        for s in range(tile_steps):
            slot = s & 1
            r.run(pcs[f"abc_s{slot}_v{1 if s == 0 else 0}"])
            r.run(pcs[f"d_s{slot}"])
        assert r.mfma - before == tile_steps * 4 * live * tn
        r.lds_done = r.lds_issued                  # the epilogue drains the LDS queue; vector loads stay in flight
        r.vm_issued += 24                          # ... and issues stores of its own: waits only get stricter
    # the first step of a tile starts the sums, every later one adds to them
    first = [ln for ln in pcs["abc_s0_v1"] if ln.startswith("MFMA")]
    assert all(ln.endswith(", 0") for ln in first[:live * tn])
    assert not any(ln.endswith(", 0") for ln in first[live * tn:])
    assert not any(ln.endswith(", 0") for ln in pcs["abc_s0_v0"] if ln.startswith("MFMA"))


def test_generated_text_names_only_planned_registers():
    gen = _load()
    text = gen.generate()
    assert text == gen.generate()
    for m in re.finditer(r"\bv\[(\d+):(\d+)\]", text):
        lo, hi = int(m.group(1)), int(m.group(2))
        assert hi < 64 or lo >= 128, m.group(0)     # fragments or stages, never the compiler's v64..v127
    for word in ("s_store", "s_buffer_store", "s_atomic", "s_dcache", "v_pk_"):
        assert word not in text
