"""Parity of the fp8 x fp8 expert path: e4m3 weights AND per-row e4m3
activations, multiplied on the fp8 matrix pipe (``dice_quantize_fp8_act``,
``dice_grouped_mlp_a8`` and ``act_quant`` of the layer call).

The reference has no fp8 code (its experts are models.py:252-273 in fp16/fp32);
the quantisation scheme is defined by this build and restated in the oracle
(``quantize_fp8_act``, ``Fp8ActExpert``).  Bars:

* quantiser: bytes and scales bit-exact against the oracle;
* expert MLP against the oracle with the SAME quantisation: 1e-2 relative L2
  (aggregate and 5x per row).  It cannot be exact: the matrix pipe's fp8
  accumulation and the oracle's fp32 sums round differently, a flipped last
  bf16 bit of ``h`` may flip an e4m3 code of fc2's input;
* whole block against the bf16 master weights: 5e-2 over all tokens.
"""
import copy

import pytest
import torch

from oracle import dice_oracle as O
from tests.helpers import block_from_params, check_rows, rel_l2

pytestmark = pytest.mark.gpu

SAME_QUANT_TOL, FP8_TOL = 1e-2, 5e-2


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from dice_amd import lib
    lib.load()
    return torch.device("cuda:0")


def _gen(seed):
    return torch.Generator().manual_seed(seed)


def _bias_params(p, seed, dtype=torch.bfloat16):
    g = _gen(seed)
    for e in list(p.experts) + ([p.shared] if p.shared is not None else []):
        e.fc1_b = (torch.randn(e.fc1_b.shape, generator=g) * 0.1).to(dtype)
        e.fc2_b = (torch.randn(e.fc2_b.shape, generator=g) * 0.1).to(dtype)
    return p


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("cols", [64, 384, 1152, 2048, 4608, 8192])
def test_act_quantiser_bit_exact(dev, dtype, cols):
    from dice_amd import ops
    g = _gen(cols)
    rows = 67
    x = (torch.randn(rows, cols, generator=g) * torch.logspace(-3, 2, rows)[:, None]).to(dtype)
    x[5] = 0                                   # all-zero row: scale 1, zero bytes
    x[7, 3] = 300.0                            # one outlier sets the row's scale
    q, s = ops.quantize_fp8_act(x.to(dev))
    wq, ws = O.quantize_fp8_act(x)
    assert torch.equal(s.cpu(), ws)
    assert torch.equal(q.cpu().view(torch.uint8), wq.view(torch.uint8))
    # gathered through a permutation, with a device-side row count and dropped entries
    perm = torch.randperm(rows * 2, generator=g).int()
    perm[40:] = -1
    n_rows = torch.tensor([33], dtype=torch.int32)
    q, s = ops.quantize_fp8_act(x.to(dev), perm.to(dev), 2, n_rows.to(dev))
    src = (perm[:33] // 2).long()
    assert torch.equal(q.cpu().view(torch.uint8)[:33], wq.view(torch.uint8)[src])
    assert torch.equal(s.cpu()[:33], ws[src])
    assert not q.cpu().view(torch.uint8)[33:].any() and not s.cpu()[33:].any()   # untouched


def test_act_quantiser_keeps_non_finite_rows_visible(dev):
    """A row with a NaN or an infinity gets a NaN scale (and zero bytes), so that
    every output of that row is NaN, as the 16-bit path would give; its
    neighbours are untouched.  Pinned in the oracle alike (build-defined)."""
    from dice_amd import ops
    x = torch.randn(6, 1024, generator=_gen(77)).bfloat16()
    x[1, 5] = float("nan")
    x[3, 1000] = float("inf")
    x[4, 17] = float("-inf")
    q, s = ops.quantize_fp8_act(x.to(dev))
    wq, ws = O.quantize_fp8_act(x)
    assert torch.equal(torch.isnan(s.cpu()), torch.tensor([False, True, False, True, True, False]))
    assert torch.equal(torch.isnan(ws), torch.isnan(s.cpu()))
    good = ~torch.isnan(ws)
    assert torch.equal(s.cpu()[good], ws[good])
    assert torch.equal(q.cpu().view(torch.uint8), wq.view(torch.uint8))
    # through the expert GEMMs: NaN rows out, finite neighbours
    D, E = 1024, 4
    p = O.make_block_params(D, E, 2, 2, None, seed=5, dtype=torch.bfloat16)
    blk = block_from_params(p, D, "swiglu", torch.bfloat16, dev)
    blk.quantize_fp8(activations=True)
    idx = torch.tensor([0, 1] * 6)
    w = torch.full((12, 1), 0.5).bfloat16()
    y = blk.moe_infer(x.to(dev), idx.to(dev), w.to(dev)).cpu().float()
    assert torch.isnan(y[[1, 3, 4]]).all() and torch.isfinite(y[[0, 2, 5]]).all()


def _packed(p, variant, dev):
    if variant == "swiglu":
        w1 = torch.stack([torch.cat([e.gate_proj, e.up_proj], 0) for e in p.experts])
        w2 = torch.stack([e.down_proj for e in p.experts])
        return w1.to(dev), w2.to(dev), None, None
    w1 = torch.stack([e.fc1_w for e in p.experts])
    w2 = torch.stack([e.fc2_w for e in p.experts])
    b1 = torch.stack([e.fc1_b for e in p.experts]).float()
    b2 = torch.stack([e.fc2_b for e in p.experts]).float()
    return w1.to(dev), w2.to(dev), b1.to(dev), b2.to(dev)


@pytest.mark.parametrize("variant", ["swiglu", "gelu_tanh"])
@pytest.mark.parametrize("D,ratio,E,counts", [
    (768, 4, 8, None),                                     # shortest reduction the kernel takes (six steps)
    (512, 4, 8, [0, 1, 700, 0, 257, 3, 1086, 1]),          # fc1 too short (k = 512): refused, see below
    (1024, 2, 8, [0, 1, 700, 0, 257, 3, 1086, 1]),         # empty, one-row and ragged groups
    (2048, 4, 16, None),                                   # DiT-G width
    # a group's last tile multiplies only its live 64-row blocks: every residue around the block edges
    (768, 2, 16, [63, 64, 65, 127, 128, 129, 191, 192, 193, 255, 256, 257, 320, 0, 1, 7]),
    (1024, 2, 8, [256 + 63, 256 + 64, 256 + 65, 512 + 128, 512 + 129, 256 + 191, 256 + 193, 513]),
])
def test_mlp_a8_matches_oracle(dev, variant, D, ratio, E, counts):
    """``dice_grouped_mlp_a8`` (rows gathered through the permutation by the
    quantiser) against the oracle's expert with the same quantisation, every
    row; ``h`` after stage 1 as well."""
    from dice_amd import ops
    from dice_amd.lib import DiceError
    N = 1024 if counts is None else sum(counts) // 2
    assert counts is None or sum(counts) == 2 * N
    g = _gen(77 + D)
    p = O.make_block_params(D, E, 2, ratio, n_shared=0, seed=8, dtype=torch.bfloat16, variant=variant)
    if variant == "gelu_tanh":
        _bias_params(p, 9)
    x = torch.randn(N, D, generator=g).bfloat16()
    if counts is None:
        idx = torch.randint(0, E, (N * 2,), generator=g)
    else:
        idx = torch.cat([torch.full((c,), e) for e, c in enumerate(counts)])
        idx = idx[torch.randperm(idx.numel(), generator=g)]
    _, offsets, perm, _ = O.dispatch_tables(idx, E)
    rows = idx.numel()
    w1, w2, b1, b2 = _packed(p, variant, dev)
    q1, s1 = ops.quantize_fp8_rowwise(w1)
    q2, s2 = ops.quantize_fp8_rowwise(w2)
    args = (x.to(dev), perm.int().to(dev), 2, offsets.int().to(dev), rows, q1, q2, s1, s2, variant, b1, b2)
    if D < 768:
        with pytest.raises(DiceError, match="multiples of 256"):
            ops.grouped_mlp_a8(*args)
        return
    out, h = ops.grouped_mlp_a8(*args)
    out, h = out.cpu(), h.cpu()
    xg = x[perm // 2]
    want = torch.empty(rows, D)
    want_h = torch.empty(rows, ratio * D)
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi == lo:
            continue
        ex = O.Fp8ActExpert(p.experts[e])
        # the library's weight quantiser and the oracle's agree bit for bit (tested elsewhere)
        want_h[lo:hi] = ex.hidden_act(xg[lo:hi]).float()
        want[lo:hi] = ex(xg[lo:hi]).float()
    check_rows(h, want_h, SAME_QUANT_TOL, "h after fc1")
    check_rows(out, want, SAME_QUANT_TOL, "expert rows")
    # and against the bf16 masters: the quantisation noise of four e4m3 operands
    master = torch.empty(rows, D)
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi > lo:
            master[lo:hi] = p.experts[e](xg[lo:hi]).float()
    assert 1e-2 < rel_l2(out, master) < 0.1


def _a8_oracle(p, h_blocks=False):
    p8 = copy.copy(p)
    p8.experts = [O.Fp8ActExpert(e, h_blocks=h_blocks) for e in p.experts]
    return p8


@pytest.mark.parametrize("variant,n_shared", [("swiglu", 2), ("gelu_tanh", 8)])
def test_block_c5_a8_full_size(dev, variant, n_shared):
    """DiT-G/2-like block (8192 tokens, D = 2048, E = 16, I = 8192), routed
    experts on the fp8 matrix pipe, shared expert bf16: every token against the
    bf16 masters (5e-2) and against the oracle with the same quantisation."""
    D, E = 2048, 16
    p = O.make_block_params(D, E, 2, 4, n_shared, seed=3, dtype=torch.bfloat16, variant=variant)
    if variant == "gelu_tanh":
        _bias_params(p, 4)
    x = torch.randn(32, 256, D, generator=_gen(5)).bfloat16()
    blk = block_from_params(p, D, variant, torch.bfloat16, dev)
    blk.quantize_fp8(activations=True)
    y = blk(x.to(dev)).cpu()
    want, widx, _, logits = O.sparse_moe_block_forward(p, x)       # every token, bf16 master weights
    ok = ~O.gate_tie_rows(logits, 2).view(-1)
    idx, _, _ = blk.gate(x.to(dev))
    assert torch.equal(idx.cpu()[ok], widx[ok])
    err = check_rows(y.view(-1, D)[ok], want.view(-1, D)[ok], FP8_TOL, "C5 fp8 x fp8 vs bf16 masters")
    assert err > 1e-3                                              # the quantised operands are really in use
    same, _, _, _ = O.sparse_moe_block_forward(_a8_oracle(p), x)
    check_rows(y.view(-1, D)[ok], same.view(-1, D)[ok], SAME_QUANT_TOL, "C5 fp8 x fp8 vs same quantisation")
    # the 16-bit-activation path on the same weights is a different computation
    blk.quantize_fp8(activations=False)
    y16 = blk(x.to(dev)).cpu()
    assert not torch.equal(y16, y)


@pytest.mark.parametrize("h_blocks", [False, True])
def test_block_a8_staleness_identities(dev, h_blocks):
    """Put and skip steps with fp8 activations: a put step returns the plain
    step's rows, a skip step fed its own cache reproduces them (the recomputed
    slot's rows are quantised row by row, so dropping the other slot changes
    nothing), and a zipf-loaded router with empty experts runs."""
    from dice_amd import lib
    from tests.helpers import zipf_bias
    D, E, N = 1024, 16, 1536
    p = O.make_block_params(D, E, 2, 4, 2, seed=11, dtype=torch.bfloat16, gate_bias=zipf_bias(E, 3.0))
    x = torch.randn(N, D, generator=_gen(12)).bfloat16().to(dev)
    blk = block_from_params(p, D, "swiglu", torch.bfloat16, dev)
    blk.quantize_fp8(activations=True, h_blocks=h_blocks)
    # Bit-identity needs whole fc2 tiles: by default a short last turn is cut along
    # k, a skip step has half the rows and so another cut, and sums of 16-bit pieces
    # differ from a whole tile's in the last bit (tests/test_gpu_split_turn.py).
    lib.load().dice_set_gemm_config(0, 50)
    try:
        plain = blk.run(x).clone()
        for mode in ("high", "low"):
            mask = O.skip_mask(2 * N, mode).to(dev)
            cache = torch.empty_like(x)
            put = blk.run(x, lib.MODE_PUT, mask, None, cache).clone()
            assert torch.equal(put, plain)
            skip = blk.run(x, lib.MODE_SKIP, mask, cache, None)
            assert torch.equal(skip, plain)
    finally:
        lib.load().dice_set_gemm_config(0, 0)
    # default schedule: the same identities to the rounding of the pieces
    mask = O.skip_mask(2 * N, "high").to(dev)
    cache = torch.empty_like(x)
    put = blk.run(x, lib.MODE_PUT, mask, None, cache).clone()
    assert torch.equal(put, blk.run(x))
    check_rows(blk.run(x, lib.MODE_SKIP, mask, cache, None).cpu(), put.cpu(), 4e-3, "skip step on its own cache")
    check_rows(put.cpu(), plain.cpu(), 4e-3, "cut last turn vs whole tiles")
    want, _, _, logits = O.sparse_moe_block_forward(_a8_oracle(p, h_blocks), x.cpu().view(1, N, D))
    ok = ~O.gate_tie_rows(logits, 2).view(-1)
    check_rows(plain.cpu()[ok], want.view(-1, D)[ok], SAME_QUANT_TOL, "zipf-loaded fp8 x fp8 block")


def test_act_quant_needs_fp8_weights_and_bf16(dev):
    from dice_amd.lib import DiceError
    D, E = 1024, 8
    p = O.make_block_params(D, E, 2, 4, 2, seed=1, dtype=torch.float16)
    blk = block_from_params(p, D, "swiglu", torch.float16, dev)
    with pytest.raises(DiceError, match="act_quant"):      # refused when asked for, not at the first forward
        blk.quantize_fp8(activations=True)
    # widths the fp8 matrix-pipe kernels do not take (DiT-XL: 1152 = 4.5 x 256) are refused up front as well
    p = O.make_block_params(1152, E, 2, 4, 2, seed=1, dtype=torch.bfloat16)
    blk = block_from_params(p, 1152, "swiglu", torch.bfloat16, dev)
    with pytest.raises(DiceError, match="multiple of 256"):
        blk.quantize_fp8(activations=True)
    blk.quantize_fp8()                                      # e4m3 weights with 16-bit activations still apply
    assert blk(torch.zeros(1, 64, 1152, dtype=torch.bfloat16, device=dev)).shape == (1, 64, 1152)


@pytest.mark.parametrize("h_blocks", [False, True])
def test_block_a8_one_arithmetic_behind_every_entry_point(dev, h_blocks):
    """A block that quantises its activations computes its routed experts on the
    fp8 matrix pipe whichever way it is entered: SparseMoeBlock.moe_infer
    (models.py:361-382) and moe_infer_ep (expertpara/ep_fwd.py:19) with the
    caller's own routing give the oracle's Fp8ActExpert result, the same rows
    bit for bit, and not the result of the 16-bit-activation path."""
    from dice_amd import ParaMode, diep
    from dice_amd.ep_fwd import moe_infer_ep
    D, E, N, k = 1024, 8, 600, 2
    g = _gen(31)
    p = O.make_block_params(D, E, k, 4, None, seed=30, dtype=torch.bfloat16)
    x = torch.randn(N, D, generator=g).bfloat16()
    idx = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(N)]).view(-1)
    w = torch.rand(N * k, 1, generator=g).bfloat16()
    blk = block_from_params(p, D, "swiglu", torch.bfloat16, dev, para_mode=ParaMode(ep=True))
    blk.quantize_fp8(activations=True, h_blocks=h_blocks)
    want = O.moe_infer(x, _a8_oracle(p, h_blocks).experts, idx, w, k)
    y = blk.moe_infer(x.to(dev), idx.to(dev), w.to(dev)).cpu()
    check_rows(y, want, SAME_QUANT_TOL, "moe_infer on the fp8 matrix pipe vs same quantisation")
    diep.ep_cache_init(cache_capacity=1, noskip_step=1)
    y_ep = moe_infer_ep(x.to(dev), blk.experts, idx.to(dev), w.to(dev), k, False).cpu()
    assert torch.equal(y_ep, y)
    blk.quantize_fp8(activations=False)
    y16 = blk.moe_infer(x.to(dev), idx.to(dev), w.to(dev)).cpu()
    assert not torch.equal(y16, y)


@pytest.mark.parametrize("h_blocks", [False, True])
def test_block_a8_step_lag_and_fused_caller(dev, h_blocks):
    """The fp8 x fp8 experts behind the other two layer entry points: a
    displaced (step-lagged) call returns, bit for bit, what the synchronous
    fp8 block produced two steps earlier, and the fused-caller call equals
    LayerNorm / modulate -> the same block -> gated residual done by hand."""
    import torch.nn.functional as F
    from dice_amd import ParaMode, diep
    D, E, N = 1024, 8, 1024
    p = O.make_block_params(D, E, 2, 4, None, seed=21, dtype=torch.bfloat16)
    sync = block_from_params(p, D, "swiglu", torch.bfloat16, dev)
    sync.quantize_fp8(activations=True, h_blocks=h_blocks)
    pm = ParaMode(ep=True, ep_async=True, ep_async_mode="all")
    lag = block_from_params(p, D, "swiglu", torch.bfloat16, dev, para_mode=pm)
    lag.quantize_fp8(activations=True, h_blocks=h_blocks)
    g = _gen(22)
    xs = [torch.randn(1, N, D, generator=g).bfloat16().to(dev) for _ in range(4)]
    plain = [sync(x).clone() for x in xs]
    diep.ep_cache_init(cache_capacity=1)
    diep.use_latest_expert_weights(False)
    try:
        for t, x in enumerate(xs):
            if t == 0:
                diep.diep_force_sync()
                diep.ep_cache_clear()
            y = lag(x)
            if t == 0:
                diep.diep_cancel_sync()
            src = 0 if t < 2 else t - 2
            assert torch.equal(y, plain[src]), f"step {t} should return step {src}"
    finally:
        diep.ep_cache_init(cache_capacity=1, noskip_step=1)
        if diep.diep_forced_sync():
            diep.diep_cancel_sync()
    # fused caller: x + gate * moe(modulate(norm(x))) with the layer input rounded to bf16 in between
    B, T = 4, N // 4
    xb = xs[0].view(B, T, D)
    shift, scale, gate = ((torch.randn(B, D, generator=g) * 0.3).bfloat16().to(dev) for _ in range(3))
    got = sync.forward_modulated(xb, shift, scale, gate)
    h = (F.layer_norm(xb.float(), (D,), None, None, 1e-6) * (1 + scale.float().unsqueeze(1))
         + shift.float().unsqueeze(1)).bfloat16()
    want = xb.float() + gate.float().unsqueeze(1) * sync(h).float()
    assert rel_l2(got.float().cpu(), want.cpu()) < 5e-3          # one bf16 rounding of the sum apart


# --------------------------------------------------------------------------- #
# h quantised inside fc1's epilogue: one power-of-two scale per row and 32 columns
# --------------------------------------------------------------------------- #
def _mlp_case(variant, D, ratio, E, counts, dev, seed=8):
    from dice_amd import ops
    N = 1024 if counts is None else sum(counts) // 2
    g = _gen(177 + D)
    p = O.make_block_params(D, E, 2, ratio, n_shared=0, seed=seed, dtype=torch.bfloat16, variant=variant)
    if variant == "gelu_tanh":
        _bias_params(p, 9)
    x = torch.randn(N, D, generator=g).bfloat16()
    if counts is None:
        idx = torch.randint(0, E, (N * 2,), generator=g)
    else:
        idx = torch.cat([torch.full((c,), e) for e, c in enumerate(counts)])
        idx = idx[torch.randperm(idx.numel(), generator=g)]
    _, offsets, perm, _ = O.dispatch_tables(idx, E)
    w1, w2, b1, b2 = _packed(p, variant, dev)
    q1, s1 = ops.quantize_fp8_rowwise(w1)
    q2, s2 = ops.quantize_fp8_rowwise(w2)
    args = (x.to(dev), perm.int().to(dev), 2, offsets.int().to(dev), idx.numel(), q1, q2, s1, s2, variant, b1, b2)
    return p, x, perm, offsets, args


H_BLOCK_CASES = [
    ("swiglu", 768, 4, 8, None),
    ("gelu_tanh", 768, 4, 8, None),
    ("swiglu", 1024, 2, 8, [0, 1, 700, 0, 257, 3, 1086, 1]),          # empty, one-row and ragged groups
    ("gelu_tanh", 1024, 2, 8, [0, 1, 700, 0, 257, 3, 1086, 1]),
    ("swiglu", 2048, 4, 16, None),                                     # DiT-G width
    # a group's last tile multiplies only its live 64-row blocks: residues around the block edges
    ("swiglu", 768, 2, 16, [63, 64, 65, 127, 128, 129, 191, 192, 193, 255, 256, 257, 320, 0, 1, 7]),
    ("gelu_tanh", 1024, 2, 8, [256 + 63, 256 + 64, 256 + 65, 512 + 128, 512 + 129, 256 + 191, 256 + 193, 513]),
]


@pytest.mark.parametrize("variant,D,ratio,E,counts", H_BLOCK_CASES)
def test_fc1_epilogue_block_quantiser_bit_exact(dev, variant, D, ratio, E, counts):
    """fc1 with ``h_blocks`` against the oracle's block quantiser applied to the
    bf16 ``h`` the same kernel writes without it (same sums, same order, the
    quantiser starts from the value rounded to bf16): bytes and exponents of
    every row, bit for bit."""
    from dice_amd import ops
    p, x, perm, offsets, args = _mlp_case(variant, D, ratio, E, counts, dev)
    rows, inter = args[4], ratio * D
    _, h16 = ops.grouped_mlp_a8(*args, stages=1)
    h8 = torch.zeros((rows, inter), dtype=torch.bfloat16, device=dev)
    ops.grouped_mlp_a8(*args, stages=1, h=h8, h_blocks=True)
    q, e = ops.split_h_blocks(h8, rows, inter)
    want_q, want_e = O.quantize_fp8_act_blocks(h16.cpu())
    assert torch.equal(e.cpu(), want_e)
    assert torch.equal(q.cpu(), want_q.view(torch.uint8))
    # the scales do their work: blocks of one row differ in exponent
    assert (want_e.max(dim=1).values > want_e.min(dim=1).values).any()


@pytest.mark.parametrize("variant,D,ratio,E,counts", H_BLOCK_CASES)
def test_fc2_on_block_scaled_rows(dev, variant, D, ratio, E, counts):
    """fc2 alone on block-scaled e4m3 rows made by the oracle - exponents spread
    over 40 powers of two within a row, so a scale applied to the wrong block,
    k-block or lane half shows - against the oracle's product of the dequantised
    rows; then the whole MLP against ``Fp8ActExpert(h_blocks=True)``."""
    from dice_amd import ops
    p, x, perm, offsets, args = _mlp_case(variant, D, ratio, E, counts, dev)
    rows, inter = args[4], ratio * D
    g = _gen(5 + D)
    h = torch.randn(rows, inter, generator=g)
    h = h * torch.exp2(torch.randint(-20, 20, (rows, inter // 32), generator=g).float()).repeat_interleave(32, dim=1)
    q, e = O.quantize_fp8_act_blocks(h.bfloat16())
    hbuf = torch.zeros((rows, inter), dtype=torch.bfloat16, device=dev)
    ops.join_h_blocks(hbuf, q.view(torch.uint8).to(dev), e.to(dev))
    out, _ = ops.grouped_mlp_a8(*args, stages=2, h=hbuf, h_blocks=True)
    hd = O.dequantize_fp8_act_blocks(q, e)
    want = torch.empty(rows, D)
    for ex in range(E):
        lo, hi = int(offsets[ex]), int(offsets[ex + 1])
        if hi > lo:
            o8 = O.Fp8ActExpert(p.experts[ex])
            w = (hd[lo:hi] @ o8.q2.float().t()) * o8.s2[None, :]
            want[lo:hi] = (w + o8.b2 if o8.b2 is not None else w).bfloat16().float()
    check_rows(out.cpu(), want, SAME_QUANT_TOL, "fc2 on block-scaled rows")
    # both stages
    out, _ = ops.grouped_mlp_a8(*args, h_blocks=True)
    xg = x[perm // 2]
    want = torch.empty(rows, D)
    for ex in range(E):
        lo, hi = int(offsets[ex]), int(offsets[ex + 1])
        if hi > lo:
            want[lo:hi] = O.Fp8ActExpert(p.experts[ex], h_blocks=True)(xg[lo:hi]).float()
    check_rows(out.cpu(), want, SAME_QUANT_TOL, "expert rows, h in blocks")


def test_block_quantiser_special_blocks(dev):
    """All-zero blocks, a block with an infinity, amax exactly 448 x 2^n and tiny values, through fc1's
    epilogue: arranged with GELU experts whose fc1 weights are zero, so that h = gelu(bias)."""
    from dice_amd import ops
    D, ratio, E = 768, 2, 8
    p, x, perm, offsets, args = _mlp_case("gelu_tanh", D, ratio, E, None, dev)
    args = list(args)
    rows, inter = args[4], ratio * D
    b1 = torch.zeros(E, inter)
    b1[:, 32:64] = 448.0                       # gelu(448) = 448: amax / 448 a power of two
    b1[:, 64:96] = torch.linspace(-3, 3, 32)
    b1[:, 96:128] = 1e-3
    b1[:, 128:160] = 56.0
    b1[3, 160] = float("inf")
    b1[:, 192:224] = torch.randn(E, 32, generator=_gen(1)) * 100
    args[5] = torch.zeros_like(args[5])        # fc1 weights: e4m3 zeros
    args[10] = b1.to(dev)
    h16 = ops.grouped_mlp_a8(*args, stages=1)[1]
    h8 = torch.zeros((rows, inter), dtype=torch.bfloat16, device=dev)
    ops.grouped_mlp_a8(*args, stages=1, h=h8, h_blocks=True)
    q, e = ops.split_h_blocks(h8, rows, inter)
    want_q, want_e = O.quantize_fp8_act_blocks(h16.cpu())
    assert torch.equal(e.cpu(), want_e) and torch.equal(q.cpu(), want_q.view(torch.uint8))
    lo, hi = int(offsets[3]), int(offsets[4])
    assert hi > lo and (q.cpu()[lo:hi, 160:192] == 0x7F).all() and (e.cpu()[lo:hi, 5] == 127).all()
    assert (e.cpu()[:, 0] == 0).all() and (q.cpu()[:, :32] == 0).all()
    assert (e.cpu()[:, 1] == 127).all() or (e.cpu()[:, 1] == 128).all()


@pytest.mark.parametrize("variant,n_shared", [("swiglu", 2), ("gelu_tanh", 8)])
def test_block_c5_h_blocks_full_size(dev, variant, n_shared):
    """The DiT-G/2-like block with ``quantize_fp8(activations=True, h_blocks=True)``: every token against the
    bf16 masters (5e-2), against the oracle with the same quantisation, and no further from the masters than
    the per-row form."""
    D, E = 2048, 16
    p = O.make_block_params(D, E, 2, 4, n_shared, seed=3, dtype=torch.bfloat16, variant=variant)
    if variant == "gelu_tanh":
        _bias_params(p, 4)
    x = torch.randn(32, 256, D, generator=_gen(5)).bfloat16()
    blk = block_from_params(p, D, variant, torch.bfloat16, dev)
    blk.quantize_fp8(activations=True, h_blocks=True)
    y = blk(x.to(dev)).cpu()
    want, _, _, logits = O.sparse_moe_block_forward(p, x)
    ok = ~O.gate_tie_rows(logits, 2).view(-1)
    err = check_rows(y.view(-1, D)[ok], want.view(-1, D)[ok], FP8_TOL, "C5, h in blocks, vs bf16 masters")
    p8 = copy.copy(p)
    p8.experts = [O.Fp8ActExpert(e, h_blocks=True) for e in p.experts]
    same, _, _, _ = O.sparse_moe_block_forward(p8, x)
    check_rows(y.view(-1, D)[ok], same.view(-1, D)[ok], SAME_QUANT_TOL, "C5, h in blocks, vs same quantisation")
    blk.quantize_fp8(activations=True)
    y_rows = blk(x.to(dev)).cpu()
    err_rows = rel_l2(y_rows.view(-1, D)[ok], want.view(-1, D)[ok])
    assert not torch.equal(y_rows, y) and err < 1.05 * err_rows
    # the routed-experts entry of the module computes what the layer call does
    blk.quantize_fp8(activations=True, h_blocks=True)
    idx, wt, _ = blk.gate(x.to(dev))
    assert blk._desc is None or blk._desc.act_quant == 2


def test_h_blocks_refuses_a_call_with_more_tiles_than_its_table_holds(dev):
    """fc2 on block-scaled rows has no variant that rebuilds its tile table (64 tiles per workgroup):
    a call that would need it is refused before anything is launched, and the per-row form takes it."""
    from dice_amd.lib import DiceError
    D, E, N = 768, 8, 736 * 1024            # (2 N / 256 + 8) x 3 tiles over 256 workgroups: 67 each
    p = O.make_block_params(D, E, 2, 1, None, seed=2, dtype=torch.bfloat16)
    blk = block_from_params(p, D, "swiglu", torch.bfloat16, dev)
    blk.quantize_fp8(activations=True, h_blocks=True)
    x = torch.zeros(1, N, D, dtype=torch.bfloat16, device=dev)
    with pytest.raises(DiceError, match="act_quant 2"):
        blk(x)
    y = blk(x[:, :4096])
    assert y.shape == (1, 4096, D) and torch.isfinite(y).all()
