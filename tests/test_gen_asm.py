"""The generated k-loop of the expert GEMM (dice_amd/csrc/gen_persist64_asm.py): what the
generator must guarantee whatever its schedule, checked on the text it writes (no GPU).

An independent replay of every statement sequence the kernel runs (prologue, then tiles of
steps) with in-order LDS and vector-memory queues: every MFMA reads fragments whose LDS reads
have completed under the waits in the text AND that hold the k-block, slot and row / weight
block its accumulator calls for (fragments replaced in place included), every LDS write sends a
stage register whose load has completed, no load refills a stage register before the LDS write
that reads it was issued, and every register stays inside the plan the build-time checker
assumes.
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

    def __init__(self, kind_desc):
        self.k = kind_desc
        self.f8 = bool(kind_desc.get("f8"))
        self.scaled = bool(kind_desc.get("scaled"))
        self.scale_slot_written = [False, False]
        self.lds_issued = self.lds_done = 0
        self.vm_issued = self.vm_done = 0
        self.frag_ready = {}      # first register of a 16-byte fragment part -> index of the LDS read filling it
        self.frag_tag = {}        # ... -> (operand, slot, address index, byte offset) it was read from
        self.stage_ready = {}     # first register of a stage entry -> index of the load filling it
        self.stage_sent = {}      # first register of a stage entry -> True once its LDS write was issued
        self.mfma = 0
        self.blocks = []          # (slot, k-block) of every MFMA, in order

    def _operand(self, first_reg, n_parts, operand, block_offset):
        """The (slot, address indices) the parts of a fragment were read from; checks readiness and offsets."""
        tags = []
        for part in range(n_parts):
            r = first_reg + 4 * part
            assert r in self.frag_ready, f"fragment v{r} never read"
            assert self.frag_ready[r] < self.lds_done, f"fragment v{r} still in flight"
            op, slot, kk, off = self.frag_tag[r]
            assert op == operand and off == block_offset, (r, self.frag_tag[r], operand, block_offset)
            tags.append((slot, kk))
        return tags

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
            elif op in ("MFMA", "MFMA8", "MFMA8S"):
                assert (op != "MFMA") == self.f8 and (op == "MFMA8S") == self.scaled
                parts = 2 if self.f8 else 1
                scale_args = None
                if self.scaled:       # ..., C, weights' scale, activations' scale op_sel:[0,kb,0] op_sel_hi:[0,0,0]
                    m = re.fullmatch(r"v(\d+) op_sel:\[0,([01]),0\] op_sel_hi:\[0,0,0\]", ",".join(args[5:]))
                    assert m and args[4] == "v127", ln
                    scale_args = (int(m.group(1)), int(m.group(2)))
                    args = args[:4]
                (fa, a0, a1), (_, w0, w1), (_, r0, r1) = _regs(args[0]), _regs(args[1]), _regs(args[2])
                assert fa == "a" and a1 - a0 == 15 and a0 % 16 == 0 and a1 < 256
                assert w1 - w0 == 4 * parts - 1 and r1 - r0 == 4 * parts - 1 and w1 < 64 and r1 < 64
                assert args[3] in ("0", args[0])
                blk = a0 // 16 - self.k["acc0"]
                i, j = divmod(blk, self.k["TN"])
                assert 0 <= i < 4 and 0 <= j < self.k["TN"]
                tw = self._operand(w0, parts, "b", self.k["brow"][j] * 128)
                ta = self._operand(r0, parts, "a", i * 64 * 128)
                assert tw == ta, f"{ln}: operands of different k-blocks {tw} {ta}"
                if self.f8:      # address index kk = 2 kb + t
                    assert tw[0][0] == tw[1][0] and tw[0][1] % 2 == 0 and tw[1][1] == tw[0][1] + 1, tw
                    self.blocks.append((tw[0][0], tw[0][1] // 2))
                    if self.scaled:
                        # the scale register holds this row block's scales of the fragments' slot, its read
                        # has completed, and op_sel picks the fragments' k-block
                        reg, byte = scale_args
                        assert self.frag_ready[reg] < self.lds_done, f"{ln}: scales still in flight"
                        assert self.frag_tag[reg] == ("s", tw[0][0], i) and byte == tw[0][1] // 2, ln
                else:
                    self.blocks.append(tw[0])
                self.mfma += 1
            elif op == "ds_read_b128":
                _, d0, d1 = _regs(args[0])
                assert d1 - d0 == 3 and d1 < 64
                m = re.fullmatch(r"%\[r([ab])(\d)(\d)\] offset:(\d+)", args[1])
                assert m, ln
                self.frag_ready[d0] = self.lds_issued
                self.frag_tag[d0] = (m.group(1), int(m.group(2)), int(m.group(3)), int(m.group(4)))
                self.lds_issued += 1
            elif op == "ds_read_u16":
                m = re.fullmatch(r"v(\d+)", args[0])
                m2 = re.fullmatch(r"%\[rs\] offset:(\d+)", args[1])
                assert self.scaled and m and m2, ln
                reg, off = int(m.group(1)), int(m2.group(1))
                slot, i = divmod(off, 1024)
                assert i % 256 == 0 and reg == 119 + 4 * slot + i // 256 and slot < 2 and i // 256 < 4, ln
                # (the slot's table must hold the step's scales: sent there by an LDS write issued earlier)
                assert self.scale_slot_written[slot], f"{ln}: the slot's scales were never written"
                self.frag_ready[reg] = self.lds_issued
                self.frag_tag[reg] = ("s", slot, i // 256)
                self.lds_issued += 1
            elif op == "ds_write_b32":
                m = re.fullmatch(r"%\[wrs\]", args[0])
                m2 = re.fullmatch(r"v(\d+) offset:(\d+)", args[1])
                assert self.scaled and m and m2, ln
                reg, off = int(m2.group(1)), int(m2.group(2))
                assert reg in (117, 118) and off == 1024 * (reg - 117), ln
                assert reg in self.stage_ready and self.stage_ready[reg] < self.vm_done, f"{ln}: load in flight"
                self.stage_sent[reg] = True
                self.scale_slot_written[reg - 117] = True
                self.lds_issued += 1
            elif op == "buffer_load_dword":
                m = re.fullmatch(r"v(\d+)", args[0])
                assert self.scaled and m and int(m.group(1)) in (117, 118), ln
                assert [a.split(" ")[0] for a in args[1:]] == ["%[vs]", "%[dS]", "%[kso]"], ln
                reg = int(m.group(1))
                assert self.stage_sent.get(reg, True), f"{ln}: refilled before it was sent to LDS"
                self.stage_ready[reg] = self.vm_issued
                self.stage_sent[reg] = False
                self.vm_issued += 1
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


@pytest.mark.parametrize("kind", [0, 1, 2, 3, 4, 5, 6, 7])
@pytest.mark.parametrize("live", [1, 2, 3, 4])
def test_generated_loop_waits_cover_every_dependence(kind, live):
    gen = _load()
    pcs = gen.simulate(kind, live)
    tn = gen.KINDS[kind]["TN"]
    assert sorted(pcs) == ["abc_s0_v0", "abc_s0_v1", "abc_s1_v0", "d_s0", "d_s1", "load_q0_stage1",
                           "load_step0", "load_step1", "read_first", "write_q0_stage1", "write_step0"]
    r = Replay(gen.KINDS[kind])
    f8 = bool(gen.KINDS[kind].get("f8"))
    per_step = (2 if f8 else 4) * live * tn    # products per step: two k-blocks of 64 (fp8) or four of 16
    for name in ("load_step0", "load_step1", "write_step0", "load_step0", "write_q0_stage1", "load_q0_stage1"):
        r.run(pcs[name])
    r.lds_done = r.lds_issued                      # s_waitcnt lgkmcnt(0) + barrier in the kernel's own code
    for tile_steps in (6, 18, 8):                  # (even step counts of at least six, as the launcher admits)
        r.run(pcs["read_first"])
        before = r.mfma
        r.blocks = []
        for s in range(tile_steps):
            slot = s & 1
            r.run(pcs[f"abc_s{slot}_v{1 if s == 0 else 0}"])
            r.run(pcs[f"d_s{slot}"])
        assert r.mfma - before == tile_steps * per_step
        # the k-blocks in order: every step its slot, its blocks one after the other, each live * tn products
        n_kb = 2 if f8 else 4
        want = [(s & 1, kb) for s in range(tile_steps) for kb in range(n_kb) for _ in range(live * tn)]
        assert r.blocks == want
        r.lds_done = r.lds_issued                  # the epilogue drains the LDS queue; vector loads stay in flight
        r.vm_issued += 24                          # ... and issues stores of its own: waits only get stricter
    # the first step of a tile starts the sums, every later one adds to them
    def starts(ln):      # the product's C operand is the constant 0
        return ln.split(",")[3].strip() == "0"
    first = [ln for ln in pcs["abc_s0_v1"] if ln.startswith("MFMA")]
    assert all(starts(ln) for ln in first[:live * tn])
    assert not any(starts(ln) for ln in first[live * tn:])
    # every block of sums is started exactly once per tile
    started = sorted(ln.split(",")[0] for ln in first[:live * tn])
    assert len(set(started)) == live * tn
    assert not any(starts(ln) for ln in pcs["abc_s0_v0"] if ln.startswith("MFMA"))


def test_generated_text_names_only_planned_registers():
    gen = _load()
    text = gen.generate()
    assert text == gen.generate()
    for m in re.finditer(r"\bv\[(\d+):(\d+)\]", text):
        lo, hi = int(m.group(1)), int(m.group(2))
        assert hi < 64 or lo >= 128, m.group(0)     # fragments or stages, never the compiler's v64..v127
    # single registers: only the scaled kind's (its kernel leaves v117..v127 to the text)
    singles = {int(m.group(1)) for m in re.finditer(r"\bv(\d+)\b", text)}
    assert singles and singles <= set(range(117, 128)), singles
    # every instruction of the text is one of these (the replay above refuses anything else, too)
    allowed = {"s_waitcnt", "s_barrier", "ds_read_b128", "ds_write_b128", "buffer_load_dwordx4", "DICE_MFMA16",
               "DICE_MFMA8", "DICE_MFMA8_SCALED", "ds_read_u16", "ds_write_b32", "buffer_load_dword"}
    for m in re.finditer(r'^\s*"(?:" )?([A-Za-z_0-9]+)', text, re.M):
        assert m.group(1) in allowed, m.group(0)


def _fake_asm(kernel, lines):
    return "\n".join([f"{kernel}:", *lines, "\ts_endpgm", ""])


def test_register_check_flags_compiler_code_in_the_assemblys_registers(tmp_path):
    """dice_amd/check_acc_regs.py on synthetic device assembly: compiler-generated instructions
    (outside the inline-assembly markers) must stay out of the registers the kernels' assembly
    owns; the same instructions inside the markers are the assembly's own."""
    from dice_amd.check_acc_regs import check
    k4_256 = "_ZN4dice12_GLOBAL__N_120gemm_persist_kernel4ILi0ELb0ELi256ELb1ELb0ELb0EEEvNS_12PersistBatchE"
    k4_192 = "_ZN4dice12_GLOBAL__N_120gemm_persist_kernel4ILi2ELb1ELi192ELb0ELb0ELb0EEEvNS_12PersistBatchE"
    k4a = "_ZN4dice12_GLOBAL__N_121gemm_persist_kernel4aILi0ELi256ELb1ELb0ELb0EEEvNS_12PersistBatchE"
    kf8 = "_ZN4dice12_GLOBAL__N_123gemm_persist_kernel_f8aILi0ELb0ELb0EEEvNS_12PersistBatchE"
    inside = ["\t;;#ASMSTART", "\tv_mfma_f32_32x32x16_bf16 a[240:255], v[0:3], v[16:19], a[240:255]",
              "\tbuffer_load_dwordx4 v[252:255], v70, s[8:11], s72 offen", "\t;;#ASMEND"]
    ok = {
        k4_256: inside + ["\tv_add_u32_e32 v200, 4, v200"],                 # all vector registers are the compiler's here
        k4_192: inside + ["\tv_accvgpr_write_b32 a63, v9"],                 # twelve-block tiles leave a0..a63 to the compiler
        k4a: inside + ["\tv_add_u32_e32 v127, 4, v64", "\tds_read_b128 v[100:103], v90"],
        kf8: inside + ["\tv_lshlrev_b32_e32 v5, 7, v95"],
    }
    bad = {
        k4_256: ["\tv_accvgpr_write_b32 a3, v9"],
        k4_192: ["\tv_accvgpr_read_b32 v9, a64"],
        k4a: ["\tv_mov_b32_e32 v128, v5"],
        kf8: ["\tv_accvgpr_write_b32 a0, v5"],
    }
    path = tmp_path / "ok.s"
    path.write_text("".join(_fake_asm(k, v) for k, v in ok.items()))
    assert check(str(path)) == 4
    for kernel, extra in bad.items():
        path = tmp_path / "bad.s"
        path.write_text(_fake_asm(kernel, ok[kernel] + extra))
        with pytest.raises(RuntimeError, match="registers that belong to the kernel's assembly"):
            check(str(path))
    # a tuple that only reaches into the owned range counts too
    path.write_text(_fake_asm(k4a, ["\tds_read_b128 v[126:129], v90"]))
    with pytest.raises(RuntimeError):
        check(str(path))
    # a translation unit without any checked kernel is an error of the build, not a pass
    path.write_text("_Z5otherv:\n\ts_endpgm\n")
    with pytest.raises(RuntimeError, match="no checked kernel"):
        check(str(path))
