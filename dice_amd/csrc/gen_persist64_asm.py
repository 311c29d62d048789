"""Generates ``persist64_asm.inc``: the k-loop of the 64-k expert GEMM kernel
(csrc/grouped_gemm_persist.hip) as inline assembly on fixed registers.

Why assembly: the kernel keeps 256 sums per lane in the accumulation registers,
two register stages of operand data in flight and two buffers of MFMA
fragments - the whole register file.  Left to the compiler, any second copy of
the loop (a variant that multiplies only the live rows of a group's last tile,
a first step that starts the sums) or any branch inside it makes the register
allocator shuffle values through accumulation registers, and makes its
wait-count pass fall back to waiting for everything at every join.  Here every
instruction of a step, its registers and its waits are written out.

Register plan of a wave (fixed numbers):
  v[0:31], v[32:63]     fragment buffers 0 / 1: weight blocks j at +4 j, row blocks
                        i at +16 + 4 i (16 bytes per lane each)
  v[128:191], v[192:255] register stages 0 / 1: load l of a step at +4 l (named in the
                         text only: the compiler's own budget ends at v127)
  a[..]                 the sums: block (i, j) at 16 (ACC0 + i TN + j)
  everything else (addresses, descriptors) comes in as asm operands.

A step s multiplies LDS slot S = s % 2 in four blocks of 16 k.  Blocks A, B, C
(one asm statement) write quarters 1..3 of register stage S^1 (the data of step
s + 1) to slot S^1 and refill them with the loads of step s + 3.  The compiled
code between the statements moves the load side on, possibly into the next
tile.  The second statement opens with the workgroup barrier; block D then
reads the first fragments of step s + 1, writes quarter 0 of stage S (step
s + 2) to slot S and refills it with quarter 0 of step s + 4.

Kinds 0, 1, 4, 5, 6 are the 16-bit shapes (SwiGLU fc1 on 256 weight rows, fc2 on 192
and on 128, GELU fc1 on 256, SwiGLU fc1 on 128).  Kinds 2 and 3 are the kernel for fp8 activations and weights
(grouped_gemm_persist_f8.hip): the same stages, slots and quarters, but a step
is 128 k in two k-blocks of 64, a fragment is 32 bytes per lane (two LDS reads)
and there is one set of eight fragments in v[0:63] (weight block j at 8 j, row
block i at 32 + 8 i), each replaced in place by the next k-block's as soon as
its last product has been issued; the first statement of a step is k-block 0
and the first weight block of k-block 1, the second the barrier and the rest.

Kind 7 is kind 3 for activations that carry one power-of-two scale (a byte: the
exponent, biased by 127) per row and 32 k: the scaled form of the instruction
multiplies the first 16 bytes that the two lanes of a row hold by the scale of
the lane in 0-31 and their second 16 bytes by the scale of the lane 32 on.  A
step's scales - four bytes per row, ordered [lane half][k-block] - travel as a
17th load of the register stage (v117 / v118: one dword per lane, row
64 wave + lane) into 1 KB behind each LDS slot's own table, and are read two
bytes per lane and row block (ds_read_u16: the lane half's bytes of both
k-blocks, `op_sel` picks the k-block's) into v[119 + 4 slot + i] with the first
fragments of their step; v127 holds the weights' scale (1.0 in every byte).  The
statements take their own parameter list (p64s_... functions).  Nothing but the
build-time check of the device assembly keeps the compiler out of v117 .. v127:
it allocates from v0 upwards and stays below them in the variants that are built.

The script simulates the instruction stream of the prologue and a few steps,
finds for every instruction the memory operations it depends on, and emits
``s_waitcnt`` with the exact number of younger operations that may still be
outstanding (LDS operations and vector loads each complete in order).
Foreign operations issued by compiler-generated code between the statements
can only make such a wait stricter, never too lax.

Usage: python gen_persist64_asm.py [out.inc] (dice_amd/build.py calls generate()).
"""
from __future__ import annotations

KINDS = {
    # kind: (TN, copies of B per step, B frag row offsets (rows), acc block 0, B loads that use the second descriptor)
    0: dict(name="fc1 SwiGLU, 256 weight rows", TN=4, CB=8, brow=[0, 32, 128, 160], acc0=0, up_from=4),
    1: dict(name="fc2, 192 weight rows", TN=3, CB=6, brow=[0, 32, 64], acc0=4, up_from=99),
    4: dict(name="fc2, 128 weight rows", TN=2, CB=4, brow=[0, 32], acc0=8, up_from=99),
    5: dict(name="GELU fc1, 256 weight rows", TN=4, CB=8, brow=[0, 32, 64, 96], acc0=0, up_from=99),
    6: dict(name="fc1 SwiGLU, 128 weight rows", TN=2, CB=4, brow=[0, 64], acc0=8, up_from=2),
    # fp8 activations and weights (grouped_gemm_persist_f8.hip): a step is 128 k in two halves of 64 k
    2: dict(name="fp8 SwiGLU fc1, 256 weight rows", TN=4, CB=8, brow=[0, 32, 128, 160], acc0=0, up_from=4, f8=True),
    3: dict(name="fp8 GELU fc1 / fc2, 256 weight rows", TN=4, CB=8, brow=[0, 32, 64, 96], acc0=0, up_from=99, f8=True),
    7: dict(name="fp8 fc2 on block-scaled activations", TN=4, CB=8, brow=[0, 32, 64, 96], acc0=0, up_from=99, f8=True,
            scaled=True),
}
SC_STAGE, SC_REG, SC_UNIT = 117, 119, 127   # registers of the scaled kind (see the docstring)
CA = 8            # loads of activation rows per wave per step
TM = 4
LGKM_MAX, VM_MAX = 15, 63


def quarter_first(cb, q):
    return q * (CA // 2) if q <= 2 else (CA + (cb + 1) // 2 if q == 3 else CA + cb)


def side_slot(idx, n, mf, phase):
    return min(mf - 1, ((4 * idx + phase) * mf) // (4 * n))


class Stream:
    """An instruction stream with in-order LDS and vector-memory queues."""

    def __init__(self, kind, live):
        self.k = KINDS[kind]
        self.live = live
        self.lds_issued = 0       # LDS operations issued so far
        self.vm_issued = 0
        self.lds_done = 0         # operations known complete (after the last wait)
        self.vm_done = 0
        self.frag_op = {}         # fragment register base -> index of the LDS read that fills it
        self.stage_op = {}        # stage register base -> index of the load that fills it
        self.out = None           # lines of the statement being recorded (None: simulate only)
        self.waits = {}           # (statement key, site) -> minimal count seen
        self.needed = set()       # sites that had to wait in at least one place of the stream
        self.key = None
        self.site = 0

    # ---- recording ----
    def begin(self, key):
        self.key, self.site, self.out = key, 0, []

    def end(self):
        lines, self.out = self.out, None
        return lines

    def emit(self, text):
        if self.out is not None:
            self.out.append(text)

    def wait(self, kind, need_done):
        """All operations of queue `kind` up to index need_done (exclusive) must be complete."""
        issued = self.lds_issued if kind == "lgkm" else self.vm_issued
        done = self.lds_done if kind == "lgkm" else self.vm_done
        site = (self.key, self.site)
        self.site += 1
        n = issued - need_done
        cap = LGKM_MAX if kind == "lgkm" else VM_MAX
        n = max(0, min(n, cap))
        # the same statement runs in several places of the stream: keep the strictest count, and
        # emit the wait if any place needs it (what the simulation assumes complete is then a lower bound)
        prev = self.waits.get(site)
        self.waits[site] = n if prev is None else min(prev, n)
        if need_done > done:
            self.needed.add(site)
            if kind == "lgkm":
                self.lds_done = max(self.lds_done, issued - n)
            else:
                self.vm_done = max(self.vm_done, issued - n)
        self.emit(("WAIT", kind, site))

    # ---- instructions ----
    def frag_reg(self, buf, which, idx):
        return 32 * buf + (4 * idx if which == "w" else 16 + 4 * idx)

    def read_frag(self, slot, kk, buf, which, idx):
        reg = self.frag_reg(buf, which, idx)
        if which == "w":
            off = self.k["brow"][idx] * 128
            addr = f"%[rb{slot}{kk}]"
        else:
            off = idx * 64 * 128
            addr = f"%[ra{slot}{kk}]"
        self.emit(f"ds_read_b128 v[{reg}:{reg + 3}], {addr} offset:{off}")
        self.frag_op[reg] = self.lds_issued
        self.lds_issued += 1

    def n_loads(self):
        return CA + self.k["CB"] + (1 if self.k.get("scaled") else 0)

    def qfirst(self, q):
        """First load of quarter q of a step (the scales' load rides at the end of the last quarter)."""
        return quarter_first(self.k["CB"], q) if q < 4 else self.n_loads()

    def write(self, stage, l):
        if l == CA + self.k["CB"]:
            reg = SC_STAGE + stage
            if reg in self.stage_op:
                self.wait("vm", self.stage_op[reg] + 1)
            self.emit(f"ds_write_b32 %[wrs], v{reg} offset:{1024 * stage}")
            self.lds_issued += 1
            return
        reg = 128 + 64 * stage + 4 * l
        if reg in self.stage_op:
            self.wait("vm", self.stage_op[reg] + 1)
        i = l if l < CA else l - CA
        off = (0 if l < CA else 256 * 128) + i * 32 * 128
        self.emit(f"ds_write_b128 %[wr{stage}], v[{reg}:{reg + 3}] offset:{off}")
        self.lds_issued += 1

    def load(self, stage, l):
        if l == CA + self.k["CB"]:
            reg = SC_STAGE + stage
            self.emit(f"buffer_load_dword v{reg}, %[vs], %[dS], %[kso] offen")
            self.stage_op[reg] = self.vm_issued
            self.vm_issued += 1
            return
        reg = 128 + 64 * stage + 4 * l
        if l < CA:
            self.emit(f"buffer_load_dwordx4 v[{reg}:{reg + 3}], %[va{l}], %[dA], %[koff] offen")
        else:
            # (weight tiles are always whole - the launcher only takes widths the tile divides - so the
            # row of a load can sit in the scalar offset, which the range check does not see)
            i = l - CA
            desc = "%[dB1]" if i >= self.k["up_from"] else "%[dB0]"
            self.emit(f"buffer_load_dwordx4 v[{reg}:{reg + 3}], %[vb], {desc}, %[sb{i}] offen")
        self.stage_op[reg] = self.vm_issued
        self.vm_issued += 1

    def mfma(self, buf, i, j, first):
        tn = self.k["TN"]
        w, a = self.frag_reg(buf, "w", j), self.frag_reg(buf, "a", i)
        need = max(self.frag_op.get(w, -1), self.frag_op.get(a, -1)) + 1
        self.wait("lgkm", need)
        acc = 16 * (self.k["acc0"] + i * tn + j)
        c = "0" if first else f"a[{acc}:{acc + 15}]"
        self.emit(f"MFMA a[{acc}:{acc + 15}], v[{w}:{w + 3}], v[{a}:{a + 3}], {c}")

    # ---- fp8 kinds: fragments of 32 bytes per lane (two LDS reads), one set of eight, replaced in place ----
    def frag_reg8(self, which, idx):
        return 8 * idx if which == "w" else 32 + 8 * idx

    def read_half8(self, slot, kb, which, idx, t):
        """16-byte half t of fragment (which, idx) of k-block kb of slot `slot`."""
        reg = self.frag_reg8(which, idx) + 4 * t
        if which == "w":
            off = self.k["brow"][idx] * 128
            addr = f"%[rb{slot}{kb * 2 + t}]"
        else:
            off = idx * 64 * 128
            addr = f"%[ra{slot}{kb * 2 + t}]"
        self.emit(f"ds_read_b128 v[{reg}:{reg + 3}], {addr} offset:{off}")
        self.frag_op[reg] = self.lds_issued
        self.lds_issued += 1

    def read_scale(self, slot, i):
        reg = SC_REG + 4 * slot + i
        self.emit(f"ds_read_u16 v{reg}, %[rs] offset:{1024 * slot + 256 * i}")
        self.frag_op[reg] = self.lds_issued
        self.lds_issued += 1

    def mfma8(self, i, j, first, slot, kb):
        w, a = self.frag_reg8("w", j), self.frag_reg8("a", i)
        regs = [w, w + 4, a, a + 4]
        sc = SC_REG + 4 * slot + i
        if self.k.get("scaled"):
            regs.append(sc)
        need = max(self.frag_op.get(r, -1) for r in regs) + 1
        self.wait("lgkm", need)
        acc = 16 * (self.k["acc0"] + i * self.k["TN"] + j)
        c = "0" if first else f"a[{acc}:{acc + 15}]"
        if self.k.get("scaled"):
            self.emit(f"MFMA8S a[{acc}:{acc + 15}], v[{w}:{w + 7}], v[{a}:{a + 7}], {c}, v{SC_UNIT}, v{sc} "
                      f"op_sel:[0,{kb},0] op_sel_hi:[0,0,0]")
        else:
            self.emit(f"MFMA8 a[{acc}:{acc + 15}], v[{w}:{w + 7}], v[{a}:{a + 7}], {c}")

    def column(self, j, up):
        rows = range(self.live) if up else range(self.live - 1, -1, -1)
        return [(i, j) for i in rows]

    def run8(self, prods, first_n, n_block, slot, kb, rslot, rkb, carried, wstage, quarters, scales=()):
        """The products `prods` in order, the first first_n of them starting the sums.  The first n_block of them
        are one k-block; behind the last product of that block that uses a fragment come the two reads that
        replace it by the fragment of k-block rkb of slot rslot (`carried` = fragments already free when the
        statement starts); products past n_block use the new fragments.  The quarters' LDS writes and refills
        are spread over all gaps.  (slot, kb): the k-block of the first n_block products; `scales`: row blocks
        whose scales of slot rslot are read behind the first product."""
        cb = self.k["CB"]
        mf = len(prods)
        gaps = [[] for _ in range(mf)]
        last_w, last_a = {}, {}
        for m, (i, j) in enumerate(prods[:n_block]):
            last_w[j] = m
            last_a[i] = m
        frees = [(0, f) for f in carried]
        frees += [(m, ("w", j)) for j, m in last_w.items()]
        frees += [(m, ("a", i)) for i, m in last_a.items()]
        for g, (which, idx) in sorted(frees):
            # (both halves before the first product past the block, which may be the fragment's next user)
            gaps[min(g, n_block - 1)].append(("r", (which, idx, 0)))
            gaps[min(g + 1, n_block - 1)].append(("r", (which, idx, 1)))
        for i in scales:
            gaps[0].append(("s", i))
        items = [l for q in quarters for l in range(self.qfirst(q), self.qfirst(q + 1))]
        for n, l in enumerate(items):
            gaps[side_slot(n, len(items), mf, 1)].append(("w", l))
        for n, l in enumerate(items):
            gaps[side_slot(n, len(items), mf, 3)].append(("l", l))
        for g in range(mf):
            i, j = prods[g]
            if g < n_block:
                self.mfma8(i, j, g < first_n, slot, kb)
            else:
                self.mfma8(i, j, g < first_n, rslot, rkb)
            for kind in ("r", "s", "w", "l"):
                for k2, x in gaps[g]:
                    if k2 != kind:
                        continue
                    if kind == "r":
                        self.read_half8(rslot, rkb, x[0], x[1], x[2])
                    elif kind == "s":
                        self.read_scale(rslot, x)
                    elif kind == "w":
                        self.write(wstage, x)
                    else:
                        self.load(wstage, x)

    def frags8(self):
        return [("w", j) for j in range(self.k["TN"])] + [("a", i) for i in range(self.live)]

    def abc8(self, slot, var):
        """First statement of an fp8 step: the 64-k block kb = 0 (weight block by weight block, the row blocks up
        and down in turn), its fragments replaced in place by those of kb = 1 as they die; then the first weight
        block of kb = 1 (the rows downwards: the order in which their fragments arrived).  Quarters 1..3 of the
        next step go from register stage slot^1 to LDS slot slot^1 and are refilled."""
        first = 4 * self.live if var == 1 else 0
        half0 = [p for j in range(4) for p in self.column(j, j % 2 == 0)]
        self.run8(half0 + self.column(0, False), first, len(half0), slot, 0, slot, 1, [], slot ^ 1, (1, 2, 3))

    def d8(self, slot):
        """Second statement: the barrier, then weight blocks 1..3 of kb = 1, the fragments replaced by those of the
        next step's kb = 0 (other slot); quarter 0 of the step after next goes to this slot and is refilled."""
        self.needed.add((self.key, self.site))
        self.wait("lgkm", self.lds_issued)
        self.emit("s_barrier")
        prods = [p for j in (1, 2, 3) for p in self.column(j, j % 2 == 1)]
        # weight block 0 of kb = 1 had its last product in the first statement
        scales = range(self.live) if self.k.get("scaled") else ()
        self.run8(prods, 0, len(prods), slot, 1, slot ^ 1, 0, [("w", 0)], slot, (0,), scales)

    # ---- the pieces ----
    def frag_order(self):
        tn = self.k["TN"]
        return [("w", 0), ("a", 0)] + [("w", j) for j in range(1, tn)] + [("a", i) for i in range(1, self.live)]

    def block(self, mbuf, rslot, rkk, wstage, q, var):
        """Products of fragment buffer mbuf; reads of (rslot, rkk) into the other buffer;
        quarter q of stage wstage to its slot, then refilled."""
        tn, cb = self.k["TN"], self.k["CB"]
        prods = [(i, ((tn - 1 - m) if (i & 1) else m)) for i in range(self.live) for m in range(tn)]
        if var == 2:
            prods = []
        reads = self.frag_order()
        f, e = self.qfirst(q), self.qfirst(q + 1)
        items = list(range(f, e))
        mf = max(1, len(prods))
        gaps = [[] for _ in range(mf)]
        for n, r in enumerate(reads):
            gaps[side_slot(n, len(reads), mf, 0)].append(("r", r))
        for n, l in enumerate(items):
            gaps[side_slot(n, len(items), mf, 1)].append(("w", l))
        for n, l in enumerate(items):
            gaps[side_slot(n, len(items), mf, 3)].append(("l", l))
        for g in range(mf):
            if prods:
                i, j = prods[g]
                self.mfma(mbuf, i, j, var == 1)
            # reads first: a read queued behind a write waits for the write's 16 cycles
            for kind in ("r", "w", "l"):
                for k2, x in gaps[g]:
                    if k2 != kind:
                        continue
                    if kind == "r":
                        self.read_frag(rslot, rkk, mbuf ^ 1, x[0], x[1])
                    elif kind == "w":
                        self.write(wstage, x)
                    else:
                        self.load(wstage, x)

    def abc(self, slot, var):
        if self.k.get("f8"):
            return self.abc8(slot, var)
        self.block(0, slot, 1, slot ^ 1, 1, var)
        self.block(1, slot, 2, slot ^ 1, 2, 0 if var == 1 else var)
        self.block(0, slot, 3, slot ^ 1, 3, 0 if var == 1 else var)

    def d(self, slot, var):
        if self.k.get("f8"):
            return self.d8(slot)
        # This wave has read slot `slot` for the last time and finished writing the other one;
        # after the barrier both hold for every wave.  (The barrier opens this statement rather
        # than closing the one before: the scalar bookkeeping between the two then runs while the
        # LDS queue drains, not after the barrier with the matrix pipe idle.)
        self.needed.add((self.key, self.site))
        self.wait("lgkm", self.lds_issued)
        self.emit("s_barrier")
        self.block(1, slot ^ 1, 0, slot, 0, 0 if var == 1 else var)

    def load_step(self, stage):
        for l in range(self.n_loads()):
            self.load(stage, l)

    def write_step(self, stage):
        for l in range(self.n_loads()):
            self.write(stage, l)

    def quarter(self, stage, q, what):
        for l in range(self.qfirst(q), self.qfirst(q + 1)):
            (self.write if what == "w" else self.load)(stage, l)

    def read_first(self):
        if self.k.get("f8"):
            for which, idx in self.frags8():
                for t in (0, 1):
                    self.read_half8(0, 0, which, idx, t)
            if self.k.get("scaled"):
                for i in range(self.live):
                    self.read_scale(0, i)
            return
        for which, idx in self.frag_order():
            self.read_frag(0, 0, 0, which, idx)


def render(lines, waits, needed):
    out = []
    for ln in lines:
        if isinstance(ln, tuple):
            _, kind, site = ln
            if site in needed:
                out.append(f"s_waitcnt {'lgkmcnt' if kind == 'lgkm' else 'vmcnt'}({waits[site]})")
        else:
            out.append(ln)
    return out


def simulate(kind, live):
    """Runs the kernel's instruction stream: prologue, a tile of 8 steps (first step starting the
    sums), a tile restart as after an epilogue, 8 more steps.  Returns {name: lines}."""
    pieces = {}
    st = Stream(kind, live)

    def rec(name, fn, *args):
        st.begin(name)
        fn(*args)
        lines = st.end()
        if name in pieces:
            assert [x for x in pieces[name] if not isinstance(x, tuple)] == \
                   [x for x in lines if not isinstance(x, tuple)], name
        pieces[name] = lines

    # prologue (as gemm_persist64_body): steps 0 and 1 through the stages into the slots (of step 1 only
    # the first quarter), steps 2 and 3 (first quarter) into the stages behind them
    rec("load_step0", st.load_step, 0)
    rec("load_step1", st.load_step, 1)
    rec("write_step0", st.write_step, 0)
    rec("load_step0", st.load_step, 0)
    rec("write_q0_stage1", st.quarter, 1, 0, "w")
    rec("load_q0_stage1", st.quarter, 1, 0, "l")
    st.lds_done = st.lds_issued           # s_waitcnt lgkmcnt(0) + barrier in the host code
    for tile in range(3):
        rec("read_first", st.read_first)
        for s in range(8):
            slot = s & 1
            var = 1 if s == 0 else 0
            rec(f"abc_s{slot}_v{var}", st.abc, slot, var)
            rec(f"d_s{slot}", st.d, slot, 0)
        # the epilogue: LDS traffic of the host code, drained; vector loads stay in flight
        st.lds_done = st.lds_issued
    # the variant of a first step whose sums do not start from zero (biased tiles) is the plain one: v0 of slot 0
    # appears from step 2 on; make sure both exist
    assert "abc_s0_v0" in pieces and "abc_s0_v1" in pieces and "abc_s1_v0" in pieces
    return {name: render(lines, st.waits, st.needed) for name, lines in pieces.items()}


def c_string(lines):
    return "\n".join(f'      "{ln}\\n"' for ln in lines)


def generate() -> str:
    out = ["// Generated by gen_persist64_asm.py - do not edit.  See that script for the register plan,",
           "// the order of the pieces and how the wait counts are derived.",
           "#pragma once"]
    # (the scaled kind's statements take more operands: a function family of their own)
    for fam, macro, scaled in (("p64", "P64", False), ("p64s", "P64S", True)):
        names = None
        table = {}
        for kind in KINDS:
            if bool(KINDS[kind].get("scaled")) != scaled:
                continue
            for live in range(1, TM + 1):
                pcs = simulate(kind, live)
                table[(kind, live)] = pcs
                names = sorted(pcs)
        for name in names:
            out.append(f"template <int KIND, int LIVE>\n__device__ __forceinline__ void {fam}_{name}({macro}_PARAMS) {{")
            first = True
            for (kind, live), pcs in table.items():
                text = [ln.replace("MFMA8S", '" DICE_MFMA8_SCALED "').replace("MFMA8 ", '" DICE_MFMA8 " ')
                        .replace("MFMA ", '" DICE_MFMA16 " ') for ln in pcs[name]]
                cond = f"KIND == {kind} && LIVE == {live}"
                out.append(f"  {'if' if first else 'else if'} constexpr ({cond})")
                out.append("    asm volatile(")
                out.append(c_string(text) if text else '      ""')
                out.append(f"      {macro}_CONSTRAINTS);")
                first = False
            out.append("  else static_assert(KIND < 0, \"no such variant\");\n}")
    return "\n".join(out) + "\n"


if __name__ == "__main__":
    import sys
    if len(sys.argv) > 1:
        with open(sys.argv[1], "w") as f:
            f.write(generate())
    else:
        sys.stdout.write(generate())
