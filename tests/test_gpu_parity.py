"""Parity of the HIP path against the CPU oracle, through the C ABI.

Bars: indices / permutations / counts bit-exact (router indices except on rows
the oracle marks as logit near-ties <= 1e-6); fp32 outputs within 1e-4, bf16
within 2e-2 and fp8 within 5e-2 relative L2.
"""
import os

import numpy as np
import pytest
import torch

from oracle import dice_oracle as O
from tests.helpers import block_from_params, check_rows, rel_l2, whole_fc2_tiles, zipf_bias

pytestmark = pytest.mark.gpu

FP32_TOL, BF16_TOL, FP8_TOL = 1e-4, 2e-2, 5e-2


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from dice_amd import lib
    lib.load()
    return torch.device("cuda:0")


def _gen(seed):
    return torch.Generator().manual_seed(seed)


# --------------------------------------------------------------------------- #
# router
# --------------------------------------------------------------------------- #
def _check_gate(dev, x, w, k, norm=False, bias=None):
    from dice_amd import ops
    want_idx, want_w, want_logits = O.gate_forward(x, w, k, norm, bias)
    idx, wt, logits, idx64 = ops.gate_topk(x.to(dev), w.to(dev), k, norm,
                                           None if bias is None else bias.to(dev),
                                           want_logits=True, want_int64=True)
    idx, wt, logits, idx64 = idx.cpu(), wt.cpu(), logits.cpu(), idx64.cpu()
    assert idx64.dtype == torch.int64 and torch.equal(idx64, idx.long())
    assert torch.allclose(logits, want_logits, atol=2e-5, rtol=1e-5)
    ties = O.gate_tie_rows(want_logits, k, tol=1e-6)
    assert torch.equal(idx.long()[~ties], want_idx[~ties]), "router indices differ off the tie rows"
    assert torch.allclose(wt[~ties], want_w[~ties], atol=1e-6, rtol=1e-5)
    assert ties.float().mean() < 0.01
    return int(ties.sum())


@pytest.mark.parametrize("N,D,E,k,dtype", [
    (1024, 384, 8, 2, torch.float32),      # DiT-S/2 block
    (8192, 1152, 8, 2, torch.bfloat16),    # DiT-XL/2 block
    (8192, 2048, 16, 2, torch.bfloat16),   # DiT-G/2-like block
    (1000, 768, 16, 4, torch.float16),
    (517, 1024, 5, 3, torch.float32),      # ragged token count, odd expert count
    (3, 64, 64, 8, torch.float32),
    # 16-bit activations and router matrix, at most 32 experts: the matrix-pipe router
    (777, 1152, 7, 2, torch.bfloat16),     # ragged token count (25 column blocks, the last with 9 tokens), odd expert count
    (300, 2304, 32, 8, torch.float16),     # 32 experts, top-8, eight waves per token block
    (64, 192, 24, 3, torch.bfloat16),      # three steps per wave
    (33, 1024, 1, 1, torch.bfloat16),      # a single expert
    (100, 4096, 8, 2, torch.bfloat16),     # too long for it: the dot-product router
    (50, 72, 8, 2, torch.bfloat16),        # hidden not a multiple of 64: the dot-product router
])
def test_gate_matches_oracle(dev, N, D, E, k, dtype):
    g = _gen(N + E)
    x = torch.randn(N, D, generator=g).to(dtype)
    w = (torch.randn(E, D, generator=g) * 0.02).to(dtype)
    _check_gate(dev, x, w, k)


def test_gate_options_and_fp32_router_weights(dev):
    g = _gen(3)
    x = torch.randn(2048, 1152, generator=g).bfloat16()
    w = torch.randn(8, 1152, generator=g) * 0.02          # fp32 router for bf16 activations
    _check_gate(dev, x, w, 2, norm=True)
    _check_gate(dev, x, w, 2, bias=zipf_bias(8))
    _check_gate(dev, x, w.bfloat16(), 2, norm=True, bias=zipf_bias(8))


def test_gate_exact_ties_pick_lower_expert(dev):
    from dice_amd import ops
    x = torch.zeros(70, 64, device=dev)
    w = torch.randn(8, 64, generator=_gen(1)).to(dev)
    idx, wt, _, _ = ops.gate_topk(x, w, 2)
    assert idx.cpu().tolist() == [[0, 1]] * 70
    assert torch.allclose(wt.cpu(), torch.full((70, 2), 0.125))


def test_gate_fixture(dev, golden_dir):
    from dice_amd import ops
    z = np.load(os.path.join(golden_dir, "gate_small.npz"))
    x = torch.zeros(37, 64)
    x[:, :24] = torch.from_numpy(z["x"])          # hidden padded to a multiple of 8 with zeros
    w = torch.zeros(8, 64)
    w[:, :24] = torch.from_numpy(z["w"])
    idx, wt, logits, _ = ops.gate_topk(x.to(dev), w.to(dev), 2, want_logits=True)
    assert np.array_equal(idx.cpu().numpy(), z["idx"])
    np.testing.assert_allclose(wt.cpu().numpy(), z["weight"], rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(logits.cpu().numpy(), z["logits"], rtol=1e-5, atol=1e-5)


# --------------------------------------------------------------------------- #
# dispatch
# --------------------------------------------------------------------------- #
def _check_dispatch(dev, idx, E, mask=None):
    from dice_amd import ops
    counts, offsets, perm, inv = ops.dispatch(idx.int().to(dev), E, None if mask is None else mask.to(dev))
    counts, offsets, perm, inv = counts.cpu().long(), offsets.cpu().long(), perm.cpu().long(), inv.cpu().long()
    S = idx.numel()
    if mask is None:
        kept = torch.arange(S)
        sub = idx
    else:
        kept = (~mask).nonzero().flatten()
        sub = idx[~mask]
    wc, wo, wp, _ = O.dispatch_tables(sub, E)
    assert torch.equal(counts, wc)
    assert torch.equal(offsets, wo)
    n = kept.numel()
    assert torch.equal(perm[:n], kept[wp]), "perm differs from the stable argsort"
    assert (perm[n:] == -1).all()
    want_inv = torch.full((S,), -1, dtype=torch.long)
    want_inv[kept[wp]] = torch.arange(n)
    assert torch.equal(inv, want_inv)


@pytest.mark.parametrize("S,E", [(0, 8), (1, 8), (63, 8), (256, 8), (2048, 8), (16384, 8), (32768, 8),
                                 (16384, 16), (65536, 64), (65537, 8), (200001, 16), (300000, 256),
                                 (1000, 3)])
def test_dispatch_matches_oracle(dev, S, E):
    idx = torch.randint(0, E, (S,), generator=_gen(S + E))
    _check_dispatch(dev, idx, E)


def test_dispatch_imbalance_empty_experts_and_skip(dev):
    g = _gen(8)
    p = torch.tensor([(e + 1.0) ** -1.2 for e in range(8)])
    idx = torch.multinomial(p, 32768, replacement=True, generator=g)
    _check_dispatch(dev, idx, 8)
    idx[idx == 2] = 5
    idx[idx == 7] = 0
    _check_dispatch(dev, idx, 8)                       # experts 2 and 7 empty
    _check_dispatch(dev, torch.full((5000,), 3), 8)    # a single hot expert
    for mode in ("high", "low", "rand"):
        _check_dispatch(dev, idx, 8, O.skip_mask(32768, mode))
    big = torch.randint(0, 16, (131072,), generator=g)
    _check_dispatch(dev, big, 16, O.skip_mask(131072, "rand"))


def test_dispatch_on_reference_recipe(dev, golden_dir):
    for seed in (42, 43):
        z = np.load(os.path.join(golden_dir, f"ep_recipe_seed{seed}.npz"))
        for it in range(4):
            _check_dispatch(dev, torch.from_numpy(z[f"idx{it}"]), 8)


def test_gather_rows(dev):
    from dice_amd import ops
    g = _gen(4)
    x = torch.randn(300, 128, generator=g).bfloat16()
    idx = torch.randint(0, 8, (600,), generator=g)
    _, _, perm, _ = O.dispatch_tables(idx, 8)
    out = ops.gather_rows(x.to(dev), perm.int().to(dev), 2, 600).cpu()
    assert torch.equal(out, x[perm // 2])              # _local_dispatch, ep_fwd.py:345-347


# --------------------------------------------------------------------------- #
# combine on the reference's own recipe
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("seed", [42, 43])
def test_dispatch_combine_flow_on_reference_recipe(dev, golden_dir, seed):
    """tests/test_ep.py's data flow with the experts (nn.Linear 36->36, not an
    MLP this library implements) evaluated on the host between the HIP dispatch
    and the HIP combine; expectation = the committed float64 fixture."""
    from dice_amd import ops
    z = np.load(os.path.join(golden_dir, f"ep_recipe_seed{seed}.npz"))
    W, B = torch.from_numpy(z["expert_w"]), torch.from_numpy(z["expert_b"])
    for it in range(4):
        x = torch.from_numpy(z[f"inp{it}"])
        idx = torch.from_numpy(z[f"idx{it}"])
        w = torch.from_numpy(z[f"w{it}"])
        _, offsets, perm, inv = ops.dispatch(idx.int().to(dev), 8)
        grouped = ops.gather_rows(x.to(dev), perm, 2, 256).cpu()
        off = offsets.cpu().tolist()
        outs = torch.empty_like(grouped)
        for e in range(8):
            outs[off[e]:off[e + 1]] = torch.nn.functional.linear(grouped[off[e]:off[e + 1]], W[e], B[e])
        y = ops.combine(outs.to(dev), w.view(128, 2).to(dev), 128, 2, inv_perm=inv).cpu()
        assert torch.allclose(y, torch.from_numpy(z[f"y{it}"]).float(), atol=1e-6, rtol=1e-5)


# --------------------------------------------------------------------------- #
# grouped expert MLP
# --------------------------------------------------------------------------- #
def _packed(params, variant, dtype, dev):
    ex = params.experts
    if variant == "swiglu":
        w1 = torch.stack([torch.cat([e.gate_proj, e.up_proj], 0) for e in ex])
        w2 = torch.stack([e.down_proj for e in ex])
        return w1.to(dtype).to(dev), w2.to(dtype).to(dev), None, None
    w1 = torch.stack([e.fc1_w for e in ex])
    w2 = torch.stack([e.fc2_w for e in ex])
    b1 = torch.stack([e.fc1_b for e in ex]).float()
    b2 = torch.stack([e.fc2_b for e in ex]).float()
    return w1.to(dtype).to(dev), w2.to(dtype).to(dev), b1.to(dev), b2.to(dev)


def _check_mlp(dev, N, D, E, ratio, dtype, variant, counts=None, cfg=(0, 0), tol=None, seed=0):
    from dice_amd import lib, ops
    g = _gen(seed + N)
    p = O.make_block_params(D, E, 2, ratio, n_shared=0, seed=seed, dtype=dtype, variant=variant)
    if variant == "gelu_tanh":
        for e in p.experts:
            e.fc1_b = (torch.randn(e.fc1_b.shape, generator=g) * 0.1).to(dtype)
            e.fc2_b = (torch.randn(e.fc2_b.shape, generator=g) * 0.1).to(dtype)
    x = torch.randn(N, D, generator=g).to(dtype)
    if counts is None:
        idx = torch.randint(0, E, (N * 2,), generator=g)
    else:
        idx = torch.cat([torch.full((c,), e) for e, c in enumerate(counts)])
        idx = idx[torch.randperm(idx.numel(), generator=g)]
        assert idx.numel() == N * 2
    _, offsets, perm, _ = O.dispatch_tables(idx, E)
    w1, w2, b1, b2 = _packed(p, variant, dtype, dev)
    lib.load().dice_set_gemm_config(*cfg)
    try:
        out = ops.grouped_mlp(x.to(dev), perm.int().to(dev), 2, offsets.int().to(dev), N * 2, w1, w2,
                              variant, b1, b2, scatter_to_slots=True, n_out_rows=N * 2).cpu()
        out_grouped = ops.grouped_mlp(x.to(dev), perm.int().to(dev), 2, offsets.int().to(dev), N * 2,
                                      w1, w2, variant, b1, b2, scatter_to_slots=False).cpu()
    finally:
        lib.load().dice_set_gemm_config(0, 0)
    want = torch.empty(N * 2, D, dtype=dtype)
    xs = x[torch.arange(N * 2) // 2]
    for e in range(E):
        sel = idx == e
        if sel.any():
            want[sel] = p.experts[e](xs[sel])
    tol = tol or (FP32_TOL if dtype == torch.float32 else BF16_TOL)
    assert rel_l2(out, want) < tol, f"slot-order output off: {rel_l2(out, want)}"
    if (cfg[0] == 0 or cfg[0] >= 20) and dtype != torch.float32:
        # default selection: the grouped output comes from the persistent fc2 kernel where it applies, the
        # scattered one from the permutation-addressed kernel (another order of the same fp32 sums)
        assert rel_l2(out_grouped, out[perm]) < 4e-3
    else:
        assert torch.equal(out_grouped, out[perm]), "grouped and scattered outputs must be the same rows"
    # per-row check so that one bad tile cannot hide inside the norm
    err = (out.double() - want.double()).norm(dim=1) / want.double().norm(dim=1).clamp_min(1e-6)
    assert err.max() < 5 * tol, f"worst row {int(err.argmax())} rel err {float(err.max())}"


@pytest.mark.parametrize("variant", ["swiglu", "gelu_tanh"])
def test_mlp_fp32(dev, variant):
    _check_mlp(dev, 512, 128, 8, 4, torch.float32, variant)
    _check_mlp(dev, 1024, 384, 8, 4, torch.float32, variant)   # DiT-S/2 expert shape
    # more experts than a wavefront has lanes (the tile search walks them 64 at a
    # time), some empty, most smaller than a tile
    counts = [(e * 7) % 33 for e in range(80)]
    counts[79] += 1280 - sum(counts)
    _check_mlp(dev, 640, 128, 80, 2, torch.float32, variant, counts=counts)


@pytest.mark.parametrize("cfg", [0, 1, 2, 3, 4])   # 0: default selection; 1-4: tilings of the permutation-addressed kernels
@pytest.mark.parametrize("variant", ["swiglu", "gelu_tanh"])
def test_mlp_bf16_tilings(dev, variant, cfg):
    _check_mlp(dev, 1024, 256, 8, 4, torch.bfloat16, variant, cfg=(cfg, cfg))
    _check_mlp(dev, 600, 1152, 4, 4, torch.bfloat16, variant, cfg=(cfg, cfg))  # XL width, 4.5 n-tiles


def _check_mlp_persistent(dev, N, D, E, ratio, variant, cfg, counts=None, seed=0, dtype=torch.bfloat16):
    """The persistent kernels take contiguous grouped rows (perm = None)."""
    from dice_amd import lib, ops
    g = _gen(seed + N + D)
    p = O.make_block_params(D, E, 2, ratio, n_shared=0, seed=seed, dtype=dtype, variant=variant)
    if variant == "gelu_tanh":
        for e in p.experts:
            e.fc1_b = (torch.randn(e.fc1_b.shape, generator=g) * 0.1).to(dtype)
            e.fc2_b = (torch.randn(e.fc2_b.shape, generator=g) * 0.1).to(dtype)
    x = torch.randn(N, D, generator=g).to(dtype)
    if counts is None:
        idx = torch.randint(0, E, (N * 2,), generator=g)
    else:
        idx = torch.cat([torch.full((c,), e) for e, c in enumerate(counts)])
        idx = idx[torch.randperm(idx.numel(), generator=g)]
        assert idx.numel() == N * 2
    _, offsets, perm, _ = O.dispatch_tables(idx, E)
    xg = x[perm // 2]
    w1, w2, b1, b2 = _packed(p, variant, dtype, dev)
    lib.load().dice_set_gemm_config(cfg, cfg)
    try:
        out = ops.grouped_mlp(xg.to(dev), None, 1, offsets.int().to(dev), N * 2, w1, w2, variant, b1, b2).cpu()
    finally:
        lib.load().dice_set_gemm_config(0, 0)
    want = torch.empty(N * 2, D, dtype=dtype)
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi > lo:
            want[lo:hi] = p.experts[e](xg[lo:hi])
    tol = BF16_TOL if dtype == torch.bfloat16 else 4e-3
    assert rel_l2(out, want) < tol, f"grouped output off: {rel_l2(out, want)}"
    err = (out.double() - want.double()).norm(dim=1) / want.double().norm(dim=1).clamp_min(1e-6)
    assert err.max() < 5 * tol, f"worst row {int(err.argmax())} rel err {float(err.max())}"


@pytest.mark.parametrize("cfg", [20, 21])   # 20: 32-k eight-wave pipeline only; 21: 64-k pipeline where it applies
@pytest.mark.parametrize("variant", ["swiglu", "gelu_tanh"])
def test_mlp_bf16_persistent_kernels(dev, variant, cfg):
    _check_mlp_persistent(dev, 1024, 256, 8, 4, variant, cfg)            # k = 256: too short for 64-k steps
    _check_mlp_persistent(dev, 600, 1152, 4, 4, variant, cfg)            # XL width: 192-row fc2 tiles
    _check_mlp_persistent(dev, 700, 384, 8, 4, variant, cfg)             # k = 384: six 64-k steps, fc2 n = 384 (padded tile)
    _check_mlp_persistent(dev, 512, 640, 8, 2, variant, cfg)             # k = 640 is no multiple of 128: no persistent kernel
    # empty experts, single-row groups, a group of exactly one tile, one hot expert
    _check_mlp_persistent(dev, 512, 512, 8, 2, variant, cfg, counts=[0, 1, 256, 0, 257, 3, 507, 0])
    _check_mlp_persistent(dev, 512, 512, 8, 2, variant, cfg, counts=[1024, 0, 0, 0, 0, 0, 0, 0])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_mlp_live_row_blocks_of_a_last_tile(dev, dtype):
    """The kernels with the generated k-loop multiply only the live 64-row blocks of a
    group's last tile (and the two waves that share a tile's columns take alternate
    32-row blocks): group heights at every residue around the block edges, through
    fc1 with gathered rows and fc2 on 192-, 256- and 128-row weight tiles."""
    edges = [256 + 63, 256 + 64, 256 + 65, 512 + 127, 512 + 128, 512 + 129, 256 + 191, 256 + 193]
    tol = BF16_TOL if dtype == torch.bfloat16 else F16_TOL
    n = sum(edges)
    assert n % 2 == 0
    for fc2_cfg in (0, 54):     # 54: fc2 on 128-row weight tiles wherever a launch can take them
        _check_mlp(dev, n // 2, 1152, 8, 4, dtype, "swiglu", counts=edges, cfg=(0, fc2_cfg), tol=tol)
    _check_mlp(dev, n // 2, 1024, 8, 2, dtype, "swiglu", counts=edges, tol=tol)
    small = [1, 63, 64, 65, 191, 192, 193, 255, 256, 257, 0, 511, 512, 513, 640, 33]
    assert sum(small) % 2 == 0
    _check_mlp(dev, sum(small) // 2, 1152, 16, 2, dtype, "swiglu", counts=small, cfg=(21, 21), tol=tol)


@pytest.mark.parametrize("cfg", [0, 21])   # 0: groups of few rows take the 64-row tiles; 21: they stay on the persistent kernels
@pytest.mark.parametrize("variant", ["swiglu", "gelu_tanh"])
def test_mlp_few_rows_per_group(dev, variant, cfg):
    """Small sampling batches through the per-stage entry point: at most 128 rows
    per expert on average, both kernel families against the oracle."""
    _check_mlp(dev, 64, 1152, 8, 4, torch.bfloat16, variant, cfg=(cfg, cfg))     # 16 rows per expert
    _check_mlp(dev, 300, 768, 8, 4, torch.float16, variant, cfg=(cfg, cfg), tol=F16_TOL)
    _check_mlp(dev, 512, 1152, 8, 4, torch.bfloat16, variant, cfg=(cfg, cfg))    # exactly 128 on average
    _check_mlp(dev, 7, 512, 8, 2, torch.bfloat16, variant, cfg=(cfg, cfg), counts=[0, 1, 0, 0, 13, 0, 0, 0])


def test_mlp_bf16_biased_tiles_across_experts(dev):
    """GELU experts with non-zero biases at XL width, enough rows that every
    workgroup multiplies several tiles in a row, of different experts and
    column blocks: the 256-wide tiles start their accumulators from a bias that
    is staged one tile ahead, alternating between two buffers."""
    _check_mlp_persistent(dev, 4096, 1152, 8, 4, "gelu_tanh", 21)



# --- fp16: the dtype the reference serves its XL and G models in (sample_ddp.py:77-81,97-98) ---
F16_TOL = 4e-3   # 11-bit mantissa: the 2e-2 bar of bf16 would hide a wrong rounding


@pytest.mark.parametrize("cfg", [0, 1, 2, 4])
@pytest.mark.parametrize("variant", ["swiglu", "gelu_tanh"])
def test_mlp_f16_tilings(dev, variant, cfg):
    _check_mlp(dev, 1024, 256, 8, 4, torch.float16, variant, cfg=(cfg, cfg), tol=F16_TOL)
    _check_mlp(dev, 600, 1152, 4, 4, torch.float16, variant, cfg=(cfg, cfg), tol=F16_TOL)


@pytest.mark.parametrize("cfg", [20, 21])
@pytest.mark.parametrize("variant", ["swiglu", "gelu_tanh"])
def test_mlp_f16_persistent_kernels(dev, variant, cfg):
    _check_mlp_persistent(dev, 600, 1152, 4, 4, variant, cfg, dtype=torch.float16)
    _check_mlp_persistent(dev, 700, 384, 8, 4, variant, cfg, dtype=torch.float16)
    _check_mlp_persistent(dev, 512, 512, 8, 2, variant, cfg, counts=[0, 1, 256, 0, 257, 3, 507, 0],
                          dtype=torch.float16)


@pytest.mark.parametrize("fp8", [False, True])
def test_block_f16_full_size(dev, fp8):
    """DiT-XL/2-MoE block at its real shape in fp16 (model.half() in the
    reference), with fp16 and with fp8 expert weights."""
    D, E = 1152, 8
    p = O.make_block_params(D, E, 2, 4, 2, seed=1, dtype=torch.float16)
    x = torch.randn(32, 256, D, generator=_gen(1)).half()
    blk = block_from_params(p, D, "swiglu", torch.float16, dev)
    if fp8:
        blk.quantize_fp8()
    y = blk(x.to(dev)).cpu()
    widx, _, wlogits = O.gate_forward(x, p.gate_weight, 2)
    idx, _, _ = blk.gate(x.to(dev))
    ties = O.gate_tie_rows(wlogits, 2)
    assert torch.equal(idx.cpu()[~ties], widx[~ties])
    want, _, _, logits = O.sparse_moe_block_forward(p, x)       # every token
    ok = ~O.gate_tie_rows(logits, 2).view(-1)
    err = check_rows(y.view(-1, D)[ok], want.view(-1, D)[ok], FP8_TOL if fp8 else F16_TOL, "fp16 block")
    assert not fp8 or err > 1e-3        # the quantised weights are really in use


@pytest.mark.parametrize("cfg", [0, 1, 2, 3, 4])
def test_mlp_bf16_ragged_groups(dev, cfg):
    # empty experts, single-row groups, a group of exactly one tile, one hot expert
    _check_mlp(dev, 512, 256, 8, 2, torch.bfloat16, "swiglu", counts=[0, 1, 128, 0, 257, 3, 635, 0],
               cfg=(cfg, cfg))
    _check_mlp(dev, 512, 256, 8, 2, torch.bfloat16, "gelu_tanh", counts=[1024, 0, 0, 0, 0, 0, 0, 0],
               cfg=(cfg, cfg))


def test_fp8_quantiser_bit_exact(dev):
    from dice_amd import ops
    g = _gen(12)
    w = O.xavier_uniform(200, 384, g).bfloat16()
    w[7] = 0
    q, s = ops.quantize_fp8_rowwise(w.to(dev))
    wq, ws = O.quantize_fp8_rowwise(w)
    assert torch.equal(s.cpu(), ws)
    assert torch.equal(q.cpu().view(torch.uint8), wq.view(torch.uint8))
    w32 = O.xavier_uniform(64, 128, g)
    q, s = ops.quantize_fp8_rowwise(w32.view(2, 32, 128).to(dev))
    wq, ws = O.quantize_fp8_rowwise(w32)
    assert torch.equal(s.cpu().view(-1), ws)
    assert torch.equal(q.cpu().view(torch.uint8).view(64, 128), wq.view(torch.uint8))


@pytest.mark.parametrize("cfg", [0, 1, 4])
@pytest.mark.parametrize("variant", ["swiglu", "gelu_tanh"])
def test_mlp_fp8_weights(dev, variant, cfg):
    from dice_amd import lib, ops
    N, D, E, ratio = 768, 512, 4, 4
    g = _gen(20)
    p = O.make_block_params(D, E, 2, ratio, n_shared=0, seed=5, dtype=torch.bfloat16, variant=variant)
    x = torch.randn(N, D, generator=g).bfloat16()
    idx = torch.randint(0, E, (N * 2,), generator=g)
    _, offsets, perm, _ = O.dispatch_tables(idx, E)
    w1, w2, b1, b2 = _packed(p, variant, torch.bfloat16, dev)
    q1, s1 = ops.quantize_fp8_rowwise(w1)
    q2, s2 = ops.quantize_fp8_rowwise(w2)
    lib.load().dice_set_gemm_config(cfg, cfg)
    try:
        out = ops.grouped_mlp(x.to(dev), perm.int().to(dev), 2, offsets.int().to(dev), N * 2, q1, q2,
                              variant, b1, b2, s1, s2, scatter_to_slots=True, n_out_rows=N * 2).cpu()
    finally:
        lib.load().dice_set_gemm_config(0, 0)
    # (a) against the oracle run on the de-quantised weights: only bf16 round-off remains
    d1 = O.dequantize_fp8_rowwise(q1.cpu().view(-1, q1.shape[-1]), s1.cpu().view(-1)).view(w1.shape)
    d2 = O.dequantize_fp8_rowwise(q2.cpu().view(-1, q2.shape[-1]), s2.cpu().view(-1)).view(w2.shape)
    xs = x[torch.arange(N * 2) // 2].float()
    want_q = torch.empty(N * 2, D)
    want_m = torch.empty(N * 2, D)
    inter = ratio * D
    for e in range(E):
        sel = idx == e
        if variant == "swiglu":
            want_q[sel] = O.moe_mlp(xs[sel], d1[e, :inter], d1[e, inter:], d2[e])
        else:
            want_q[sel] = O.gelu_mlp(xs[sel], d1[e], b1[e].cpu(), d2[e], b2[e].cpu())
        want_m[sel] = p.experts[e](xs[sel].bfloat16()).float()
    assert rel_l2(out, want_q) < BF16_TOL
    # (b) against the bf16 master weights: the fp8 bar
    assert rel_l2(out, want_m) < FP8_TOL


@pytest.mark.parametrize("variant", ["swiglu", "gelu_tanh"])
@pytest.mark.parametrize("D,ratio,counts", [
    (1152, 4, None),                                   # XL width: 192-wide fc2 tiles, several tiles per workgroup
    (512, 4, [0, 1, 700, 0, 257, 3, 1086, 1]),         # 256-wide fc2 tiles; empty, one-row and ragged groups
    (2048, 2, None),                                   # DiT-G width
])
def test_mlp_fp8_weights_persistent_kernel(dev, variant, D, ratio, counts):
    """fp8 weights through the 64-k persistent kernels (contiguous grouped rows):
    the bytes are widened to bf16 on their way into LDS, the per-channel scale
    multiplies the fp32 sums, and a bias enters the accumulators divided by it."""
    from dice_amd import lib, ops
    E, N = 8, 1024
    g = _gen(31 + D)
    p = O.make_block_params(D, E, 2, ratio, n_shared=0, seed=6, dtype=torch.bfloat16, variant=variant)
    if variant == "gelu_tanh":
        for e in p.experts:
            e.fc1_b = (torch.randn(e.fc1_b.shape, generator=g) * 0.1).bfloat16()
            e.fc2_b = (torch.randn(e.fc2_b.shape, generator=g) * 0.1).bfloat16()
    x = torch.randn(N, D, generator=g).bfloat16()
    if counts is None:
        idx = torch.randint(0, E, (N * 2,), generator=g)
    else:
        idx = torch.cat([torch.full((c,), e) for e, c in enumerate(counts)])
        idx = idx[torch.randperm(idx.numel(), generator=g)]
    _, offsets, perm, _ = O.dispatch_tables(idx, E)
    xg = x[perm // 2]
    w1, w2, b1, b2 = _packed(p, variant, torch.bfloat16, dev)
    q1, s1 = ops.quantize_fp8_rowwise(w1)
    q2, s2 = ops.quantize_fp8_rowwise(w2)
    lib.load().dice_set_gemm_config(21, 21)
    try:
        out = ops.grouped_mlp(xg.to(dev), None, 1, offsets.int().to(dev), N * 2, q1, q2, variant, b1, b2,
                              s1, s2).cpu()
    finally:
        lib.load().dice_set_gemm_config(0, 0)
    d1 = O.dequantize_fp8_rowwise(q1.cpu().view(-1, q1.shape[-1]), s1.cpu().view(-1)).view(w1.shape)
    d2 = O.dequantize_fp8_rowwise(q2.cpu().view(-1, q2.shape[-1]), s2.cpu().view(-1)).view(w2.shape)
    inter = ratio * D
    want = torch.empty(N * 2, D)
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi == lo:
            continue
        xs = xg[lo:hi].float()
        if variant == "swiglu":
            want[lo:hi] = O.moe_mlp(xs, d1[e, :inter], d1[e, inter:], d2[e])
        else:
            want[lo:hi] = O.gelu_mlp(xs, d1[e], b1[e].cpu(), d2[e], b2[e].cpu())
    assert rel_l2(out, want) < BF16_TOL, rel_l2(out, want)
    err = (out.double() - want.double()).norm(dim=1) / want.double().norm(dim=1).clamp_min(1e-6)
    assert err.max() < 5 * BF16_TOL, f"worst row {int(err.argmax())} rel err {float(err.max())}"


@pytest.mark.parametrize("variant,fp8", [("swiglu", False), ("gelu_tanh", False), ("swiglu", True), ("gelu_tanh", True)])
def test_persistent_kernels_rerun_bit_identical(dev, variant, fp8):
    """The persistent kernels stage tile tables, row numbers, biases and scales
    in LDS one tile ahead of their use; every workgroup multiplies several
    tiles in a row here, and twenty back-to-back launches on the same inputs
    must agree bit for bit (a buffer overwritten too early would show as a
    difference between runs)."""
    from dice_amd import lib, ops
    N, D, E, ratio = 4096, 1152, 8, 4
    g = _gen(77)
    p = O.make_block_params(D, E, 2, ratio, n_shared=0, seed=8, dtype=torch.bfloat16, variant=variant)
    if variant == "gelu_tanh":
        for e in p.experts:
            e.fc1_b = (torch.randn(e.fc1_b.shape, generator=g) * 0.1).bfloat16()
            e.fc2_b = (torch.randn(e.fc2_b.shape, generator=g) * 0.1).bfloat16()
    x = torch.randn(N * 2, D, generator=g).bfloat16().to(dev)
    idx = torch.randint(0, E, (N * 2,), generator=g)
    _, offsets, _, _ = O.dispatch_tables(idx, E)
    offsets = offsets.int().to(dev)
    w1, w2, b1, b2 = _packed(p, variant, torch.bfloat16, dev)
    s1 = s2 = None
    if fp8:
        w1, s1 = ops.quantize_fp8_rowwise(w1)
        w2, s2 = ops.quantize_fp8_rowwise(w2)
    lib.load().dice_set_gemm_config(21, 21)
    try:
        outs = [ops.grouped_mlp(x, None, 1, offsets, N * 2, w1, w2, variant, b1, b2, s1, s2) for _ in range(20)]
        torch.cuda.synchronize()
    finally:
        lib.load().dice_set_gemm_config(0, 0)
    assert all(torch.equal(o, outs[0]) for o in outs[1:])
    assert torch.isfinite(outs[0].float()).all()


# --------------------------------------------------------------------------- #
# whole block
# --------------------------------------------------------------------------- #
def _run_block(dev, p, x, variant, dtype, **kw):
    blk = block_from_params(p, x.shape[-1], variant, dtype, dev, **kw)
    return blk, blk(x.to(dev)).cpu()


@pytest.mark.parametrize("variant", ["swiglu", "gelu_tanh"])
def test_block_c1_fp32(dev, variant):
    """DiT-S/2-MoE block, fp32: x [4,256,384], E=8, top-2, I=1536, shared 2D."""
    p = O.make_block_params(384, 8, 2, 4, 2, seed=0, variant=variant)
    x = torch.randn(4, 256, 384, generator=_gen(0))
    want, widx, _, logits = O.sparse_moe_block_forward(p, x)
    blk, y = _run_block(dev, p, x, variant, torch.float32)
    assert y.shape == x.shape
    ties = O.gate_tie_rows(logits, 2)
    assert rel_l2(y.view(-1, 384)[~ties], want.view(-1, 384)[~ties]) < FP32_TOL
    idx, wt, aux = blk.gate(x.to(dev))
    assert aux is None and idx.dtype == torch.int64
    assert torch.equal(idx.cpu()[~ties], widx[~ties])
    # renormalised top-2 (the benchmark configuration's wording)
    p.norm_topk_prob = True
    want_n, _, _, _ = O.sparse_moe_block_forward(p, x)
    _, y_n = _run_block(dev, p, x, variant, torch.float32)
    assert rel_l2(y_n.view(-1, 384)[~ties], want_n.view(-1, 384)[~ties]) < FP32_TOL


def test_block_c1_fp32_pretraining_tp2(dev):
    """The reference builds its fp32 S and B models with pretraining_tp=2
    (sample_ddp.py:83): MoeMLP then slices its weights, concatenates the fc1
    halves and SUMS two partial down projections (models.py:253-269).  The
    kernels compute the unsliced product; only fc2's K-split round-off differs,
    which must stay inside the fp32 bar."""
    p = O.make_block_params(384, 8, 2, 4, 2, seed=9, pretraining_tp=2)
    assert p.experts[0].pretraining_tp == 2 and p.shared.pretraining_tp == 2
    x = torch.randn(4, 256, 384, generator=_gen(9))
    want, widx, _, logits = O.sparse_moe_block_forward(p, x)
    p1 = O.make_block_params(384, 8, 2, 4, 2, seed=9, pretraining_tp=1)
    want1, _, _, _ = O.sparse_moe_block_forward(p1, x)
    assert not torch.equal(want, want1)                # the sliced path really rounds differently
    blk = block_from_params(p, 384, "swiglu", torch.float32, dev, pretraining_tp=2)
    assert blk.experts[0].pretraining_tp == 2
    y = blk(x.to(dev)).cpu()
    ok = ~O.gate_tie_rows(logits, 2).view(-1)
    check_rows(y.view(-1, 384)[ok], want.view(-1, 384)[ok], FP32_TOL, "C1 pretraining_tp=2")
    idx, _, _ = blk.gate(x.to(dev))
    assert torch.equal(idx.cpu()[ok], widx[ok])


@pytest.mark.parametrize("N,D,E,k,dtype,tol", [
    (1024, 384, 8, 2, torch.float32, FP32_TOL),        # C1 shape
    (8192, 1152, 8, 2, torch.bfloat16, BF16_TOL),      # C2 shape
    (333, 768, 16, 4, torch.bfloat16, BF16_TOL),
])
def test_block_moe_infer_function(dev, N, D, E, k, dtype, tol):
    """SparseMoeBlock.moe_infer(x, flat_expert_indices, flat_expert_weights)
    with the reference's signature and caller-supplied routing
    (models.py:361-382): int64 indices [N*k], weights [N*k, 1] in the module
    dtype; no gate, no shared expert."""
    g = _gen(N + D + k)
    p = O.make_block_params(D, E, k, 4, 2, seed=13, dtype=dtype)
    x = torch.randn(N, D, generator=g).to(dtype)
    # k distinct experts per token, arbitrary weights (the gate is not under test)
    idx = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(N)]).view(-1)
    w = torch.rand(N * k, 1, generator=g).to(dtype)
    want = O.moe_infer(x, p.experts, idx, w, k)
    blk = block_from_params(p, D, "swiglu", dtype, dev)
    y = blk.moe_infer(x.to(dev), idx.to(dev), w.to(dev)).cpu()
    assert y.shape == (N, D) and y.dtype == dtype
    check_rows(y, want, tol, "moe_infer")


@pytest.mark.parametrize("N,D,E,k,dtype", [
    (1, 768, 8, 2, torch.bfloat16),        # a single token: seven experts empty, one-row groups
    (7, 768, 8, 2, torch.bfloat16),
    (257, 768, 16, 2, torch.bfloat16),     # DiT-B width, 16 experts, one row past a tile
    (1000, 1024, 16, 2, torch.bfloat16),   # DiT-L width
    (333, 1408, 16, 2, torch.bfloat16),    # DiT-G width (11 x 128)
    (130, 384, 8, 1, torch.float32),       # top-1
    (300, 768, 8, 1, torch.bfloat16),      # top-1 on the kernels that address rows through the permutation
    (300, 512, 4, 4, torch.float16),       # top-4 likewise
    (130, 384, 8, 4, torch.float32),       # top-4
    (64, 384, 64, 2, torch.float32),       # as many experts as the layer call takes
])
def test_block_odd_shapes(dev, N, D, E, k, dtype):
    """Token counts that fill no tile, every model width of the reference's
    configurations (models.py:769-806), other top-k and expert counts."""
    p = O.make_block_params(D, E, k, 4, 2, seed=11, dtype=dtype, gate_std=0.1)
    x = torch.randn(1, N, D, generator=_gen(N + D)).to(dtype)
    want, widx, _, logits = O.sparse_moe_block_forward(p, x)
    blk, y = _run_block(dev, p, x, "swiglu", dtype)
    ok = ~O.gate_tie_rows(logits, k)
    assert ok.float().mean() > 0.95
    assert rel_l2(y[0][ok], want[0][ok]) < (FP32_TOL if dtype == torch.float32 else BF16_TOL)
    idx, _, _ = blk.gate(x.to(dev))
    assert torch.equal(idx.cpu()[ok], widx[ok])
    # zero tokens: nothing to do, nothing launched
    empty = blk(torch.empty(1, 0, D, dtype=dtype, device=dev))
    assert empty.shape == (1, 0, D)


def _subset_oracle(p, x2d, sub, dtype):
    """Tokens are independent through the block, so the oracle on a subset of
    rows must equal the same rows of the full-size result."""
    xs = x2d[sub].to(dtype).unsqueeze(0)
    y, idx, wt, logits = O.sparse_moe_block_forward(p, xs)
    return y[0], idx, logits


@pytest.mark.parametrize("variant", ["swiglu", "gelu_tanh"])
def test_block_c2_bf16_full_size(dev, variant):
    """DiT-XL/2-MoE block at its real shape: 8192 tokens, D=1152, E=8, I=4608."""
    D, E = 1152, 8
    p = O.make_block_params(D, E, 2, 4, 2, seed=1, dtype=torch.bfloat16, variant=variant)
    x = torch.randn(32, 256, D, generator=_gen(1)).bfloat16()
    blk, y = _run_block(dev, p, x, variant, torch.bfloat16)
    # routing for every token
    widx, _, wlogits = O.gate_forward(x, p.gate_weight, 2)
    idx, _, _ = blk.gate(x.to(dev))
    ties = O.gate_tie_rows(wlogits, 2)
    assert torch.equal(idx.cpu()[~ties], widx[~ties])
    # outputs of every token, aggregate and row by row
    want, _, _, logits = O.sparse_moe_block_forward(p, x)
    ok = ~O.gate_tie_rows(logits, 2).view(-1)
    check_rows(y.view(-1, D)[ok], want.view(-1, D)[ok], BF16_TOL, f"C2 {variant}")
    # determinism: a second call is bit-identical
    assert torch.equal(blk(x.to(dev)).cpu(), y)


def test_block_many_tokens_per_workgroup(dev):
    """More tiles per workgroup than the 64-k kernel's tile table holds: the
    workgroups rewrite their table on the way.  Checked against the oracle on a
    sample and, for every token, against the same block run on quarters of the
    batch (tokens are independent and a row's sums do not depend on its tile, so
    the two must agree bit for bit)."""
    D, E, N = 384, 8, 172032
    p = O.make_block_params(D, E, 2, 4, 2, seed=5, dtype=torch.bfloat16, variant="swiglu")
    x = torch.randn(1, N, D, generator=_gen(5)).bfloat16()
    with whole_fc2_tiles():
        blk, y = _run_block(dev, p, x, "swiglu", torch.bfloat16)
        xq = x.view(4, N // 4, D).to(dev)
        parts = torch.cat([blk(xq[i:i + 1]).cpu() for i in range(4)], dim=1)
    sub = torch.randperm(N, generator=_gen(6))[:256]
    want, _, logits = _subset_oracle(p, x.view(-1, D), sub, torch.bfloat16)
    ties = O.gate_tie_rows(logits, 2).view(-1)
    assert rel_l2(y.view(-1, D)[sub][~ties], want[~ties]) < BF16_TOL
    assert torch.equal(parts.view(-1, D), y.view(-1, D))


def test_block_xl_width_large_batch_matches_chunks(dev):
    """73728 tokens at DiT-XL width: groups of ~72 m-tiles (banded tile order) and
    ~100 turns per workgroup in fc1 (rewritten tile table).  Every token must come
    out bit-identical to the same block run on 8192-token chunks, which take the
    plain tile order and a single table; a sample is checked against the oracle."""
    D, E, N = 1152, 8, 73728
    p = O.make_block_params(D, E, 2, 4, 2, seed=8, dtype=torch.bfloat16)
    x = torch.randn(1, N, D, generator=_gen(8)).bfloat16()
    with whole_fc2_tiles():
        blk, y = _run_block(dev, p, x, "swiglu", torch.bfloat16)
        xq = x.view(N // 8192, 8192, D).to(dev)
        parts = torch.cat([blk(xq[i:i + 1]).cpu() for i in range(N // 8192)], dim=1)
    assert torch.equal(parts.view(-1, D), y.view(-1, D))
    sub = torch.randperm(N, generator=_gen(9))[:128]
    want, _, logits = _subset_oracle(p, x.view(-1, D), sub, torch.bfloat16)
    ok = ~O.gate_tie_rows(logits, 2).view(-1)
    assert rel_l2(y.view(-1, D)[sub][ok], want[ok]) < BF16_TOL


@pytest.mark.parametrize("variant,dtype,fp8,N,D,ratio", [
    ("gelu_tanh", torch.bfloat16, False, 344064, 384, 4),   # biased tiles: the bias buffers are staged across a table rewrite
    ("swiglu", torch.float16, True, 172032, 384, 4),        # fp8 weights: so are the scale buffers
    ("swiglu", torch.bfloat16, "act", 180224, 768, 2),      # fp8 activations too: the fp8 kernel's scales and row scales
    ("gelu_tanh", torch.bfloat16, "act", 180224, 768, 2),   # ... and its bias
    # ... with fc1's epilogue quantising h in blocks (fc1 rewrites its table, fc2 - a quarter of the tiles - does not)
    ("swiglu", torch.bfloat16, "act_blocks", 180224, 768, 2),
    ("gelu_tanh", torch.bfloat16, "act_blocks", 180224, 768, 2),
])
def test_rewritten_tile_table_other_kernels(dev, variant, dtype, fp8, N, D, ratio):
    """The other instantiations that rewrite their tile table (more than 64 tiles
    per workgroup): every token bit-identical to the same block run on chunks
    that need no rewrite."""
    p = O.make_block_params(D, 8, 2, ratio, 2, seed=12, dtype=dtype, variant=variant)
    if variant == "gelu_tanh":
        g = _gen(13)
        for e in list(p.experts) + [p.shared]:
            e.fc1_b = (torch.randn(e.fc1_b.shape, generator=g) * 0.1).to(dtype)
            e.fc2_b = (torch.randn(e.fc2_b.shape, generator=g) * 0.1).to(dtype)
    blk = block_from_params(p, D, variant, dtype, dev)
    if fp8:
        blk.quantize_fp8(activations=fp8 in ("act", "act_blocks"), h_blocks=fp8 == "act_blocks")
    x = torch.randn(1, N, D, generator=torch.Generator(device=dev).manual_seed(14), device=dev).to(dtype)
    with whole_fc2_tiles():
        y = blk(x)
        chunk = N // 8
        parts = torch.cat([blk(x[:, i:i + chunk]) for i in range(0, N, chunk)], dim=1)
    assert torch.equal(parts, y)
    assert torch.isfinite(y.float()).all() and float(y.float().abs().max()) > 0


def test_block_c3_zipf_load(dev):
    """16384 tokens, router bias = log Zipf(1.2): heavy imbalance in the grouped GEMM."""
    D, E = 1152, 8
    p = O.make_block_params(D, E, 2, 4, 2, seed=2, dtype=torch.bfloat16, gate_bias=zipf_bias(E))
    x = torch.randn(16, 1024, D, generator=_gen(3)).bfloat16()
    blk, y = _run_block(dev, p, x, "swiglu", torch.bfloat16)
    widx, _, wlogits = O.gate_forward(x, p.gate_weight, 2, bias=p.gate_bias)
    load = torch.bincount(widx.view(-1), minlength=E).float() / widx.numel()
    assert load.max() > 0.3 and load.min() < 0.06, load
    ties = O.gate_tie_rows(wlogits, 2)
    idx, _, _ = blk.gate(x.to(dev))
    assert torch.equal(idx.cpu()[~ties], widx[~ties])
    want, _, _, logits = O.sparse_moe_block_forward(p, x)       # every token
    ok = ~O.gate_tie_rows(logits, 2).view(-1)
    check_rows(y.view(-1, D)[ok], want.view(-1, D)[ok], BF16_TOL, "C3")


def test_block_c5_fp8_full_size(dev):
    """DiT-G/2-like block: 8192 tokens, D=2048, E=16, I=8192, e4m3 routed weights
    with per-channel scales, bf16 shared expert, checked against bf16 masters."""
    D, E = 2048, 16
    p = O.make_block_params(D, E, 2, 4, 2, seed=3, dtype=torch.bfloat16)
    x = torch.randn(32, 256, D, generator=_gen(5)).bfloat16()
    blk = block_from_params(p, D, "swiglu", torch.bfloat16, dev)
    blk.quantize_fp8()
    y = blk(x.to(dev)).cpu()
    want, _, _, logits = O.sparse_moe_block_forward(p, x)       # every token, bf16 master weights
    ok = ~O.gate_tie_rows(logits, 2).view(-1)
    err = check_rows(y.view(-1, D)[ok], want.view(-1, D)[ok], FP8_TOL, "C5 fp8 weights")
    assert err > 1e-3                                            # the quantised weights are really in use


# --------------------------------------------------------------------------- #
# staleness cache
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("mode", ["high", "low", "rand"])
def test_skip_steps_follow_oracle(dev, mode):
    """Reference schedule with interval 2 over 8 steps (first step full, odd
    steps skip), x drifting by 0.05*N(0,1) per step; oracle = moe_infer_ep with
    the same mask and its own cache."""
    from dice_amd import diep
    D, E, N = 256, 8, 512
    p = O.make_block_params(D, E, 2, 4, 2, seed=4, gate_std=0.1)
    blk = block_from_params(p, D, "swiglu", torch.float32, dev, ep=True, layer_idx=0)
    g = _gen(30)
    diep.ep_cache_init(cache_capacity=1, noskip_step=2, skip_mode=mode)
    diep.ep_set_rand_mask(None)
    mask = diep.ep_skip_mask(N * 2)
    ocache = O.EPSkipCache(1)
    x = torch.randn(1, N, D, generator=g)
    pattern = []
    try:
        for i in range(8, 0, -1):
            diep.ep_set_step(i)
            if i == 8:
                diep.ep_cache_clear()
                ocache.clear()
            now = O.skip_now(True, ocache, 0, i, 2)
            assert diep.ep_skip_now(0) == now
            pattern.append(now)
            want, _, _, logits = O.sparse_moe_block_forward(p, x, skip_mask_=mask, skip_now_=now,
                                                            cache=ocache, cache_key=0)
            y = blk(x.to(dev)).cpu()
            ok = ~O.gate_tie_rows(logits, 2)
            assert rel_l2(y[0][ok], want[0][ok]) < FP32_TOL, f"step {i} skip={now}"
            x = x + 0.05 * torch.randn(1, N, D, generator=g)
    finally:
        diep.ep_cache_init(cache_capacity=1, noskip_step=1)
    assert pattern == [False, True, False, True, False, True, False, True]


def test_skip_full_size_identities(dev):
    """C4 shape (8192 x 1152, bf16).  (i) A put step returns the plain result
    bit for bit and its cache rows are the unscaled slot outputs; (ii) a skip
    step fed with that cache on the same input reproduces the plain result bit
    for bit (the recomputed slot runs the same arithmetic, the other slot is
    read back); (iii) a skip step does half the routed rows."""
    from dice_amd.lib import MODE_PLAIN, MODE_PUT, MODE_SKIP
    D, E, N = 1152, 8, 8192
    p = O.make_block_params(D, E, 2, 4, 2, seed=6, dtype=torch.bfloat16)
    blk = block_from_params(p, D, "swiglu", torch.bfloat16, dev)
    x = torch.randn(N, D, generator=_gen(7)).bfloat16().to(dev)
    plain = blk.run(x, MODE_PLAIN).clone()
    for mode in ("high", "low", "rand"):
        mask = O.skip_mask(2 * N, mode).to(dev)
        cache = torch.empty_like(x)
        put = blk.run(x, MODE_PUT, mask, None, cache).clone()
        assert torch.equal(put, plain)
        # (bit for bit with whole fc2 tiles; by default a skip step, with half the
        # rows, may cut other left-over tiles along k than the full step did)
        with whole_fc2_tiles():
            assert torch.equal(blk.run(x, MODE_PLAIN), plain)
            skip = blk.run(x, MODE_SKIP, mask, cache, None).clone()
            assert torch.equal(skip, plain)
        check_rows(blk.run(x, MODE_SKIP, mask, cache, None).cpu(), plain.cpu(), 4e-3, "skip step on its own cache")
        # a drifted input with the stale cache stays close to its own full result
        x2 = (x.float() + 0.05 * torch.randn(N, D, generator=_gen(8)).to(dev)).bfloat16()
        full2 = blk.run(x2, MODE_PLAIN).clone()
        stale = blk.run(x2, MODE_SKIP, mask, cache, None).clone()
        assert 0 < rel_l2(stale, full2) < 0.2


def test_stage_timers_ring_and_fc1_mode(dev):
    """The CudaProfiler-scope replacement: every stage timed over a run of calls, and the
    mode that brackets the fc1 launch only."""
    import ctypes
    from dice_amd.lib import check, load
    lib = load()
    p = O.make_block_params(384, 8, 2, 4, 2, seed=3, dtype=torch.bfloat16, variant="swiglu")
    x = torch.randn(2, 512, 384, generator=_gen(3)).bfloat16()
    blk, _ = _run_block(dev, p, x, "swiglu", torch.bfloat16)
    n = lib.dice_profile_stage_count()
    names = [lib.dice_profile_stage_name(i).decode() for i in range(n)]
    assert names == ["moe.gate", "moe.dispatch", "moe.gather", "moe.mlp.fc1", "moe.mlp.shared_fc1", "moe.quant_h",
                     "moe.mlp.fc2", "moe.mlp.shared_fc2", "moe.combine"]
    # stages that hold a launch on this path (16-bit weights: the shared expert rides in the routed launches)
    busy = {"moe.gate", "moe.dispatch", "moe.mlp.fc1", "moe.mlp.fc2", "moe.combine"}
    buf = (ctypes.c_float * n)()
    xd = x.view(-1, 384).to(dev)
    assert lib.dice_profile_read(buf, n) != 0           # not enabled: an error, not garbage
    check(lib.dice_profile_enable(1))
    try:
        assert lib.dice_profile_read(buf, n) != 0       # nothing recorded yet
        for _ in range(70):                             # more calls than the ring holds
            blk.run(xd)
        check(lib.dice_profile_read(buf, n))
        all_ms = list(buf)
        assert all(0.0 < v < 50.0 for i, v in enumerate(all_ms) if names[i] in busy), all_ms
        assert all(0.0 <= v < 1.0 for i, v in enumerate(all_ms) if names[i] not in busy), all_ms
        assert lib.dice_profile_read(buf, n) != 0       # the read consumed the record
        check(lib.dice_profile_enable(2))
        for _ in range(3):
            blk.run(xd)
        check(lib.dice_profile_read(buf, n))
        fc1 = names.index("moe.mlp.fc1")
        assert 0.0 < buf[fc1] < 50.0
        assert all(buf[i] == 0.0 for i in range(n) if i != fc1)
    finally:
        check(lib.dice_profile_enable(0))
