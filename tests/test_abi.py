"""CPU-side checks of the C boundary and the host logic (no kernel launches)."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "dice_moe.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dice_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from dice_amd import lib
    cdll = lib.load()
    names = _declared_symbols()
    assert len(names) >= 11
    for n in names:
        assert hasattr(cdll, n), f"{n} declared in include/dice_moe.h but not exported"
    for n in lib.EXPORTS:
        assert n in names, f"{n} bound in python but not declared in the header"
    assert cdll.dice_abi_version() == 2


def test_layer_struct_matches_header_layout():
    from dice_amd.lib import MoeLayerDesc
    # 10 int32 fields, 12 pointers, one more int32 (+ padding), naturally aligned.
    assert MoeLayerDesc.gate_w.offset == 40
    assert MoeLayerDesc.act_quant.offset == 40 + 12 * 8
    assert ctypes.sizeof(MoeLayerDesc) == 40 + 12 * 8 + 8


def test_lag_entry_and_caller_structs_match_header_layout():
    from dice_amd.lib import CallerDesc, LagEntryDesc
    # dice_moe_lag_entry_t: six pointers and an int64; dice_moe_caller_t: three pointers, int64, float (+ padding)
    assert LagEntryDesc.max_rows.offset == 48 and ctypes.sizeof(LagEntryDesc) == 56
    assert CallerDesc.tokens_per_sample.offset == 24 and CallerDesc.ln_eps.offset == 32
    assert ctypes.sizeof(CallerDesc) == 40


def test_new_entry_points_report_bad_arguments():
    from dice_amd import lib
    from dice_amd.lib import CallerDesc, LagEntryDesc, MoeLayerDesc
    cdll = lib.load()
    one = ctypes.c_void_p(16)
    rc = cdll.dice_ln_modulate(one, one, None, one, 1, 8, 64, 4, 1e-6, None)
    assert rc == -1 and b"null pointer" in cdll.dice_last_error()
    rc = cdll.dice_ln_modulate(one, one, one, one, 1, 8, 64, 0, 1e-6, None)
    assert rc == -1 and b"tokens_per_sample" in cdll.dice_last_error()
    rc = cdll.dice_ln_modulate(one, one, one, one, 1, 8, 60, 4, 1e-6, None)
    assert rc == -1 and b"16 bytes" in cdll.dice_last_error()
    rc = cdll.dice_ln_modulate(one, one, one, one, 1, 8, 1 << 16, 4, 1e-6, None)
    assert rc == -2
    rc = cdll.dice_combine_residual(one, None, one, None, None, None, None, one, None, 4, one, 1, 8, 2, 64, None)
    assert rc == -1
    d = MoeLayerDesc()
    d.hidden, d.inter, d.n_experts, d.top_k, d.act_dtype, d.w_dtype = 128, 512, 8, 2, 1, 1
    d.gate_w = d.w1 = d.w2 = 16
    rc = cdll.dice_moe_forward_modulated(ctypes.byref(d), None, one, 8, 0, None, None, None, one, None, None,
                                         one, 1 << 30, None)
    assert rc == -1
    c = CallerDesc()            # shift / scale / gate left NULL
    rc = cdll.dice_moe_forward_modulated(ctypes.byref(d), ctypes.byref(c), one, 8, 0, None, None, None, one, None,
                                         None, one, 1 << 30, None)
    assert rc == -1 and b"shift" in cdll.dice_last_error()
    e = LagEntryDesc()          # an entry without buffers
    rc = cdll.dice_moe_forward_lagged(ctypes.byref(d), None, one, 8, 0, None, ctypes.byref(e), None, None, 0, None,
                                      None, 0, None, one, None, None, one, 1 << 30, None)
    assert rc == -1 and b"lacks a buffer" in cdll.dice_last_error()
    rc = cdll.dice_moe_forward_lagged(ctypes.byref(d), None, one, 8, 1, None, None, None, None, 0, None,
                                      None, 0, None, one, None, None, one, 1 << 30, None)
    assert rc == -1 and b"skip_mask" in cdll.dice_last_error()


def test_bad_arguments_are_reported_without_touching_a_gpu():
    from dice_amd import lib
    cdll = lib.load()
    rc = cdll.dice_gate_topk(None, 0, None, 0, None, 4, 64, 8, 2, 0, None, None, None, None, None)
    assert rc == -1 and b"null pointer" in cdll.dice_last_error()
    one = ctypes.c_void_p(16)
    rc = cdll.dice_gate_topk(one, 0, one, 0, None, 4, 63, 8, 2, 0, one, None, one, None, None)
    assert rc == -1 and b"multiple of 8" in cdll.dice_last_error()
    rc = cdll.dice_gate_topk(one, 0, one, 0, None, 4, 64, 65, 2, 0, one, None, one, None, None)
    assert rc == -2
    rc = cdll.dice_dispatch(one, None, 10, 300, one, one, one, one, None, 0, None)
    assert rc == -2
    rc = cdll.dice_combine(one, None, one, None, None, one, None, one, 1, 8, 2, 64, None)
    assert rc == -1 and b"skip_mask" in cdll.dice_last_error()
    rc = cdll.dice_grouped_mlp(one, 1, None, 1, one, 8, 16, 100, 256, one, None, one, None, None, None,
                               1, 0, one, one, 0, None)
    assert rc == -2 and b"multiples of 64" in cdll.dice_last_error()
    with pytest.raises(lib.DiceError):
        lib.check(rc)


def test_cpu_tensors_are_refused():
    from dice_amd import lib, ops
    with pytest.raises(lib.DiceError, match="no CPU path"):
        ops.gate_topk(torch.zeros(4, 64), torch.zeros(8, 64), 2)


def test_module_interface_and_state_dict_keys():
    """Same constructor, sub-module names and parameter shapes as the reference
    block (models.py:280-300; key format expertpara/etrim.py:44)."""
    from dice_amd import ParaMode, SparseMoeBlock
    blk = SparseMoeBlock(128, mlp_ratio=4, num_experts=8, num_experts_per_tok=2, pretraining_tp=1,
                         layer_idx=0, total_layers=1, para_mode=ParaMode())
    sd = blk.state_dict()
    assert sd["gate.weight"].shape == (8, 128)
    for e in range(8):
        assert sd[f"experts.{e}.gate_proj.weight"].shape == (512, 128)
        assert sd[f"experts.{e}.up_proj.weight"].shape == (512, 128)
        assert sd[f"experts.{e}.down_proj.weight"].shape == (128, 512)
    assert sd["shared_experts.gate_proj.weight"].shape == (256, 128)
    assert sd["shared_experts.down_proj.weight"].shape == (128, 256)
    assert len(sd) == 1 + 8 * 3 + 3
    blk.train()
    with pytest.raises(Exception):
        blk(torch.zeros(1, 4, 128))


def test_multi_gpu_modes_are_refused():
    from dice_amd import DiceError, ParaMode
    with pytest.raises(DiceError):
        ParaMode(sp=True)
    with pytest.raises(AssertionError):
        ParaMode(ep_async=True)          # models.py:40-41: async needs ep
    pm = ParaMode(ep=True, ep_async=True, ep_async_mode="all", ep_async_warm_up=2)
    assert pm.verbose() == "DiEP" and not pm.dp and pm.ep_async_warm_up == 2


@pytest.mark.parametrize("pipeline,strategy", [(False, "all"), (True, "all"), (True, "shallow"),
                                               (True, "deep"), (True, "interleaved")])
def test_lag_bookkeeping_matches_oracle_state_machine(pipeline, strategy):
    """Host side of the step-lagged calls: which cached entry the experts run on
    and which one is returned must be the ones the oracle's restatement of the
    reference caches (diep.py:196-289) consumes.  Entries are told apart by a
    tag stored in their x tensor; the oracle's 'experts' return the tag of the
    layer that owns them, so a wrong owner shows as well."""
    from dice_amd import diep
    from oracle import dice_oracle as O
    L, E, n, d = 4, 4, 6, 2
    diep.ep_cache_init(cache_capacity=L, async_pipeline=pipeline, selective_async_strategy=strategy)
    state = O.DiepState(L, async_pipeline=pipeline, selective_async_strategy=strategy)

    class Tagger:
        """Expert stand-in: adds 1000 * (owning layer + 1) to its input."""
        def __init__(self, layer):
            self.layer = layer
        def __call__(self, x):
            return x + 1000.0 * (self.layer + 1)

    idx = torch.arange(2 * n) % E
    w = torch.ones(2 * n, 1)
    try:
        for step in range(5):
            forced = step in (0, 3)
            if forced:
                diep.diep_force_sync()
                diep.ep_cache_clear()
                state.force_sync()
                state.cache_clear()
            for l in range(L):
                if not O.layer_is_async(strategy, l, L):
                    assert not diep.layer_is_async(strategy, l, L)
                    continue
                assert diep.layer_is_async(strategy, l, L)
                tag = float(10 * step + l + 1)
                x = torch.full((n, d), tag)
                got = O.moe_infer_ep_async(state, x, [Tagger(l)] * E, idx, w, 2, True, cache_key=l)
                new = diep.LagEntry(x, E, 2, False, owner=l, copy_x=False)
                work, emit = diep.lag_roles(l, new)
                work.rows = work.x + 1000.0 * (work.owner + 1)       # what the kernel call would leave
                # the oracle returned 2 * (emitted tag + 1000 * (owner + 1)): both slots, weight 1
                assert torch.equal(got, 2 * emit.rows), (step, l)
            if forced:
                diep.diep_cancel_sync()
                state.cancel_sync()
        assert diep.ep_all2all_cached_tensors_size() > 0
        assert diep.ep_get_max_mem() > 0
    finally:
        if diep.diep_forced_sync():
            diep.diep_cancel_sync()
        diep.ep_cache_init(cache_capacity=1)


def test_skip_policy_matches_oracle():
    """dice_amd.diep mirrors the reference's control functions; the oracle's
    restatement of diep.py:61-90 is the checker."""
    from dice_amd import diep
    from oracle import dice_oracle as O
    for mode in ("high", "low"):
        diep.ep_cache_init(cache_capacity=2, noskip_step=2, skip_mode=mode)
        assert diep.ep_skip_enabled()
        assert torch.equal(diep.ep_skip_mask(64), O.skip_mask(64, mode))
    diep.ep_cache_init(cache_capacity=2, noskip_step=2, skip_mode="rand")
    diep.ep_set_rand_mask(None)
    m = diep.ep_skip_mask(64)
    assert m.view(32, 2).sum(1).eq(1).all() and diep.ep_skip_mask(64) is m

    ocache = O.EPSkipCache(2)
    for i in range(50, 0, -1):
        diep.ep_set_step(i)
        if i == 50:
            diep.ep_cache_clear()
            ocache.clear()
        for layer in (0, 1):
            now = diep.ep_skip_now(layer)
            assert now == O.skip_now(True, ocache, layer, i, 2)
            if now:
                assert diep.ep_skip_get(layer) is not None
                ocache.get(layer)
            else:
                diep.ep_skip_put(layer, torch.zeros(3))
                ocache.put(layer, torch.zeros(3))
    assert diep.ep_cached_tensors_size() == ocache.tensors_size()
    diep.ep_cache_init(cache_capacity=2, noskip_step=1)
    assert not diep.ep_skip_enabled() and not diep.ep_skip_now(0)


def test_skip_mask_slot_literals():
    """Which slot each strategy masks, written out (reference diep.py:74-79:
    'high' -> mask[::2], the slot with the higher router score; 'low' ->
    mask[1::2]).  Exchanging the two in both the oracle and the product would
    pass every symmetry test; it fails here."""
    from dice_amd import diep
    from oracle import dice_oracle as O
    T, F = True, False
    assert O.skip_mask(8, "high").tolist() == [T, F, T, F, T, F, T, F]
    assert O.skip_mask(8, "low").tolist() == [F, T, F, T, F, T, F, T]
    try:
        diep.ep_cache_init(cache_capacity=1, noskip_step=2, skip_mode="high")
        assert diep.ep_skip_mask(8).tolist() == [T, F, T, F, T, F, T, F]
        diep.ep_cache_init(cache_capacity=1, noskip_step=2, skip_mode="low")
        assert diep.ep_skip_mask(8).tolist() == [F, T, F, T, F, T, F, T]
    finally:
        diep.ep_cache_init(cache_capacity=1, noskip_step=1)


def test_forced_sync_schedule():
    from dice_amd import diep
    assert diep.ep_forced_sync(50, 50)
    assert not diep.ep_forced_sync(49, 50)
    assert diep.ep_forced_sync(48, 50, ep_async_warm_up=2)
    assert not diep.ep_forced_sync(47, 50, ep_async_warm_up=2)
    assert diep.ep_forced_sync(40, 50, strided_sync=10)
    assert diep.ep_forced_sync(2, 50, strided_sync=100, ep_async_cool_down=3)


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asked for more (or started under a multi-rank
    launcher) it says so and exits before touching a device."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for argv, env in ((["--gpus", "2"], {}), ([], {"WORLD_SIZE": "2"})):
        r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), *argv], capture_output=True, text=True,
                           env={**os.environ, **env}, timeout=300)
        assert r.returncode == 2
        assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_header_is_plain_c_and_links(tmp_path):
    """include/dice_moe.h compiles as strict C99 and a C program links against
    the library: the boundary is usable from any language with a C FFI.  The
    program only makes calls that are answered before a device is touched."""
    import shutil
    import subprocess
    from dice_amd import lib
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = tmp_path / "abi.c"
    src.write_text(r'''
#include "dice_moe.h"
#include <stdio.h>
int main(void) {
  dice_moe_layer_t layer = {0};
  dice_moe_lag_entry_t entry = {0};
  dice_moe_caller_t caller = {0};
  (void)entry; (void)caller;
  if (dice_abi_version() < 1) return 10;
  if (dice_moe_workspace_bytes(&layer, 8) == 0) return 11;
  if (dice_gate_topk(0, DICE_BF16, 0, DICE_BF16, 0, 8, 64, 8, 2, 0, 0, 0, 0, 0, 0) != DICE_ERR_BAD_ARG) return 12;
  printf("%s\n", dice_last_error());
  return 0;
}
''')
    exe = tmp_path / "abi"
    libdir = os.path.dirname(lib.LIB_PATH)
    cc = subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(root, "include"),
                         str(src), "-o", str(exe), "-L", libdir, "-ldice_moe", f"-Wl,-rpath,{libdir}"],
                        capture_output=True, text=True)
    assert cc.returncode == 0, cc.stderr
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, (run.returncode, run.stderr)
    assert "null pointer" in run.stdout


@pytest.mark.parametrize("split", [0, 1])
@pytest.mark.parametrize("tokens", [64, 1024, 8192, 16384, 65536, 140000, 300000])
@pytest.mark.parametrize("shape", ["swiglu_fc1", "swiglu_fc2", "literal_fc2", "fp8_fc2"])
def test_tile_table_bound_covers_every_xcd_split(shape, tokens, split):
    """The host decides from a bound on a workgroup's turns whether a persistent
    expert-GEMM launch may take the kernel whose LDS tile table holds 64 turns.
    The bound has to cover both ways of sharing the tiles out over the XCDs: with
    contiguous eighths of the cost, an XCD that gets only the short tiles of a
    launch whose problems differ in k walks more tiles than an eighth of every
    problem's.  Here: the bound against the device's arithmetic restated on the
    host, with every group as tall as the row bound allows."""
    import numpy as np
    from dice_amd import lib
    cdll = ctypes.CDLL(lib.LIB_PATH)
    D, I, E = 1152, 4608, 8
    if shape == "swiglu_fc1":     # routed + shared fc1, k = D for both
        rows, experts, n, k, fc2 = [2 * tokens, tokens], [E, 1], [I, I // 2], [D, D], 0
    elif shape == "swiglu_fc2":   # routed k = I, shared k = I / 2
        rows, experts, n, k, fc2 = [2 * tokens, tokens], [E, 1], [D, D], [I, I // 2], 1
    elif shape == "literal_fc2":  # shared expert of twice the routed width: k = 2 I
        rows, experts, n, k, fc2 = [2 * tokens, tokens], [E, 1], [D, D], [I, 2 * I], 1
    else:                         # fp8 routed experts: one problem
        rows, experts, n, k, fc2 = [2 * tokens], [16], [2048], [8192], 1
    a = lambda v, t: np.asarray(v, dtype=t)
    rows_a, exp_a, n_a, k_a = a(rows, np.int64), a(experts, np.int32), a(n, np.int32), a(k, np.int32)
    bound, turns = ctypes.c_int64(), ctypes.c_int64()
    cdll.dice_debug_persist_turns.argtypes = [ctypes.c_int] + [ctypes.c_void_p] * 4 + [ctypes.c_int] * 3 + \
        [ctypes.POINTER(ctypes.c_int64)] * 2
    rc = cdll.dice_debug_persist_turns(len(rows), rows_a.ctypes.data, exp_a.ctypes.data, n_a.ctypes.data,
                                       k_a.ctypes.data, fc2, 32, split, ctypes.byref(bound), ctypes.byref(turns))
    assert rc == 0
    # (one table entry stays an invalid tile, which ends the workgroup's walk)
    assert turns.value + 1 <= bound.value, f"{shape} {tokens} tokens, split {split}: {turns.value} turns, bound {bound.value}"
    assert bound.value <= 2 * turns.value + 4, "the bound should not send small launches to the rewriting kernel"
