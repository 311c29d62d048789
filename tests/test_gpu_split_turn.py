"""The fc2 launch of the layer call cuts the tiles of a short last turn along k
(each idle workgroup multiplies one piece; a small second launch adds the
pieces in fp32): the same block with the cut switched off (tuning hook,
fc2 = 50) must agree to the rounding of the 16-bit partial tiles, and both
must meet the oracle (models.py:252-273, 292-296, 302-382) at the bar of the
other block tests.

Shapes are chosen so that every XCD's run leaves a handful of tiles (at most
a third of its 32 workgroups' worth; a few dozen tiles per launch, at least
12 steps per tile): the
cut applies in every launch checked here, with even and uneven pieces, which
the tests confirm by asking for outputs that are close but not bit-identical.
"""
import copy

import pytest
import torch

from oracle import dice_oracle as O
from tests.helpers import block_from_params, check_rows, rel_l2

pytestmark = pytest.mark.gpu

BF16_TOL, F16_TOL, SAME_QUANT_TOL, FP8_TOL = 2e-2, 4e-3, 1e-2, 5e-2


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


def _whole_and_cut(blk, x):
    """The block's output with every fc2 tile multiplied whole, then with the
    default schedule."""
    from dice_amd import lib
    lib.load().dice_set_gemm_config(0, 50)
    try:
        whole = blk(x).clone()
    finally:
        lib.load().dice_set_gemm_config(0, 0)
    return whole.cpu(), blk(x).cpu()


@pytest.mark.parametrize("variant,D,ratio,E,n_shared,N,dtype", [
    ("swiglu", 768, 2, 4, 0, 1024, torch.bfloat16),      # 192-wide fc2 tiles, no shared expert: one problem per launch
    ("gelu_tanh", 768, 2, 4, 0, 1024, torch.bfloat16),   # ... with biases: added by a tile's first piece only
    ("gelu_tanh", 1024, 2, 4, 0, 1536, torch.bfloat16),  # 256-wide fc2 tiles: the bias enters through the accumulators
    ("swiglu", 1024, 3, 8, 0, 777, torch.bfloat16),      # ragged groups, 48 steps
    ("swiglu", 1152, 2, 8, 0, 1000, torch.bfloat16),     # 36 steps in pieces of 8 to 14
    ("gelu_tanh", 1152, 1, 4, 0, 900, torch.bfloat16),   # 18 steps: at most three pieces of 6
    ("swiglu", 768, 2, 4, 0, 1024, torch.float16),       # the fp16 build of the same kernels (pieces in fp16)
    ("gelu_tanh", 1024, 2, 4, 0, 1536, torch.float16),
])
def test_16bit_block_cut_last_turn(dev, variant, D, ratio, E, n_shared, N, dtype):
    p = O.make_block_params(D, E, 2, ratio, n_shared, seed=21, dtype=dtype, variant=variant)
    if variant == "gelu_tanh":
        _bias_params(p, 22, dtype)
    x = torch.randn(1, N, D, generator=_gen(23)).to(dtype)
    blk = block_from_params(p, D, variant, dtype, dev)
    whole, cut = _whole_and_cut(blk, x.to(dev))
    want, _, _, logits = O.sparse_moe_block_forward(p, x)
    ok = ~O.gate_tie_rows(logits, 2).view(-1)
    tol = BF16_TOL if dtype == torch.bfloat16 else F16_TOL
    check_rows(whole.view(-1, D)[ok], want.view(-1, D)[ok], tol, "whole tiles vs oracle")
    check_rows(cut.view(-1, D)[ok], want.view(-1, D)[ok], tol, "cut last turn vs oracle")
    assert not torch.equal(cut, whole), "the cut did not apply: the test's shape no longer exercises it"
    check_rows(cut.view(-1, D), whole.view(-1, D), tol / 5, "cut last turn vs whole tiles")


@pytest.mark.parametrize("variant", ["swiglu", "gelu_tanh"])
@pytest.mark.parametrize("activations", [False, True, "h_blocks"])
def test_fp8_block_cut_last_turn(dev, variant, activations):
    """fp8 weights (bf16 matrix pipe) and fp8 weights x fp8 activations (fp8
    matrix pipe; also with h quantised in blocks by fc1's epilogue: a piece of a
    cut tile then starts part-way into a row of block scales), shared expert in
    launches of its own (which cut theirs too)."""
    D, E, N = 1024, 8, 1280
    p = O.make_block_params(D, E, 2, 3, 2, seed=31, dtype=torch.bfloat16, variant=variant)
    if variant == "gelu_tanh":
        _bias_params(p, 32)
    x = torch.randn(1, N, D, generator=_gen(33)).bfloat16()
    blk = block_from_params(p, D, variant, torch.bfloat16, dev)
    blk.quantize_fp8(activations=bool(activations), h_blocks=activations == "h_blocks")
    whole, cut = _whole_and_cut(blk, x.to(dev))
    if activations:   # against the oracle with the same quantisation
        ref = copy.copy(p)
        ref.experts = [O.Fp8ActExpert(e, h_blocks=activations == "h_blocks") for e in p.experts]
        tol = SAME_QUANT_TOL
    else:             # against the bf16 master weights
        ref, tol = p, FP8_TOL
    want, _, _, logits = O.sparse_moe_block_forward(ref, x)
    ok = ~O.gate_tie_rows(logits, 2).view(-1)
    check_rows(whole.view(-1, D)[ok], want.view(-1, D)[ok], tol, "whole tiles vs oracle")
    check_rows(cut.view(-1, D)[ok], want.view(-1, D)[ok], tol, "cut last turn vs oracle")
    assert not torch.equal(cut, whole), "the cut did not apply: the test's shape no longer exercises it"
    check_rows(cut.view(-1, D), whole.view(-1, D), 4e-3, "cut last turn vs whole tiles")


def test_cut_turn_is_deterministic_and_leaves_the_stage_calls_alone(dev):
    """Two calls give the same bits (pieces are added in a fixed order), and a
    skip step fed its own cache still reproduces the plain step."""
    from dice_amd import lib
    D, E, N = 768, 4, 1024
    p = O.make_block_params(D, E, 2, 2, 0, seed=41, dtype=torch.bfloat16)
    x = torch.randn(N, D, generator=_gen(42)).bfloat16().to(dev)
    blk = block_from_params(p, D, "swiglu", torch.bfloat16, dev)
    a = blk.run(x).clone()
    b = blk.run(x).clone()
    assert torch.equal(a, b)
    mask = O.skip_mask(2 * N, "high").to(dev)
    cache = torch.empty_like(x)
    put = blk.run(x, lib.MODE_PUT, mask, None, cache).clone()
    assert torch.equal(put, a)
    skip = blk.run(x, lib.MODE_SKIP, mask, cache, None)
    assert rel_l2(skip, a) < 4e-3   # (half the rows: another tile count, another cut)


def test_batch_invariant_layer_multiplies_every_tile_whole(dev):
    """``dice_moe_layer_t.batch_invariant`` (``SparseMoeBlock.batch_invariant``) is the
    supported switch for callers who need a token's result not to depend on
    what else is in the call: the layer then equals the whole-tile schedule of the
    process-wide tuning hook bit for bit, a skip step fed its own cache reproduces
    the full step exactly, and a token gives the same bits in a smaller batch."""
    from dice_amd import lib
    D, E, N = 768, 4, 1024
    p = O.make_block_params(D, E, 2, 2, 0, seed=41, dtype=torch.bfloat16)
    x = torch.randn(N, D, generator=_gen(42)).bfloat16().to(dev)
    cutting = block_from_params(p, D, "swiglu", torch.bfloat16, dev)
    whole, cut = _whole_and_cut(cutting, x.view(1, N, D))
    assert not torch.equal(whole, cut)
    blk = block_from_params(p, D, "swiglu", torch.bfloat16, dev)
    blk.batch_invariant = True
    a = blk.run(x).clone()
    assert torch.equal(a.cpu(), whole.view(N, D))
    mask = O.skip_mask(2 * N, "high").to(dev)
    cache = torch.empty_like(x)
    put = blk.run(x, lib.MODE_PUT, mask, None, cache).clone()
    skip = blk.run(x, lib.MODE_SKIP, mask, cache, None)
    assert torch.equal(put, a) and torch.equal(skip, a)
    part = blk.run(x[:300].contiguous())
    assert torch.equal(part, a[:300])


@pytest.mark.parametrize("variant,n_shared,N", [
    ("swiglu", 2, 256),       # the reference's shared expert (k = 2304) beside routed tiles of 72 steps
    ("swiglu", 2, 700),       # ragged groups, the largest batch that still takes the separate launch
    ("gelu_tanh", 8, 512),    # config-literal shared expert: its fc2 tiles are twice as long as the routed ones
    ("gelu_tanh", 8, 64),
])
def test_small_batch_shared_fc2_in_its_own_launch(dev, variant, n_shared, N):
    """Small batches at DiT-XL width: the shared expert's fc2 leaves the routed
    experts' launch so that both launches cut their tiles along k.  Against the
    oracle, against the joint launch (tuning hook fc2 = 52) and against the
    forced separate launch (51: must be what the default already does)."""
    from dice_amd import lib
    D, E = 1152, 8
    p = O.make_block_params(D, E, 2, 4, n_shared, seed=41, dtype=torch.bfloat16, variant=variant)
    if variant == "gelu_tanh":
        _bias_params(p, 42)
    x = torch.randn(1, N, D, generator=_gen(43)).bfloat16()
    blk = block_from_params(p, D, variant, torch.bfloat16, dev)
    xd = x.to(dev)
    by_rule = blk(xd).cpu()
    assert torch.equal(blk(xd).cpu(), by_rule), "two runs differ"
    outs = {}
    for hook in (51, 52):
        lib.load().dice_set_gemm_config(0, hook)
        try:
            outs[hook] = blk(xd).cpu()
        finally:
            lib.load().dice_set_gemm_config(0, 0)
    assert torch.equal(by_rule, outs[51]), "the default did not launch the shared expert's fc2 on its own"
    assert not torch.equal(by_rule, outs[52])
    want, _, _, logits = O.sparse_moe_block_forward(p, x)
    ok = ~O.gate_tie_rows(logits, 2).view(-1)
    check_rows(by_rule.view(-1, D)[ok], want.view(-1, D)[ok], BF16_TOL, "separate launches vs oracle")
    check_rows(outs[52].view(-1, D)[ok], want.view(-1, D)[ok], BF16_TOL, "joint launch vs oracle")
    check_rows(by_rule.view(-1, D), outs[52].view(-1, D), BF16_TOL / 2, "separate vs joint launch")


def _slim_and_not(blk, x):
    """The block's output with the fc2 launches on 128-row weight tiles wherever they can
    take them (tuning hook fc2 = 54), then with such tiles ruled out (55)."""
    from dice_amd import lib
    try:
        lib.load().dice_set_gemm_config(0, 54)
        slim = blk(x).clone()
        lib.load().dice_set_gemm_config(0, 55)
        wide = blk(x).clone()
    finally:
        lib.load().dice_set_gemm_config(0, 0)
    return slim.cpu(), wide.cpu()


@pytest.mark.parametrize("variant,D,ratio,E,n_shared,N,dtype", [
    ("swiglu", 1152, 4, 8, 2, 1536, torch.bfloat16),      # the reference block at a mid batch: what the model picks them for
    ("swiglu", 1152, 4, 8, 2, 1000, torch.bfloat16),      # ragged groups, short last tiles of every number of live blocks
    ("gelu_tanh", 1152, 4, 8, 8, 2048, torch.bfloat16),   # config-literal: biased, shared tiles twice as long (bias staged in LDS)
    ("gelu_tanh", 768, 2, 4, 2, 1300, torch.bfloat16),
    ("swiglu", 1024, 2, 4, 2, 1280, torch.float16),       # the fp16 build; 256 | n: against the 256-row tiles
    ("gelu_tanh", 1152, 2, 8, 2, 1111, torch.float16),
])
def test_fc2_on_128_row_weight_tiles(dev, variant, D, ratio, E, n_shared, N, dtype):
    """fc2 of a joint launch in 128-row weight tiles (the kernel with the generated k-loop,
    wave tile 128 x 64): the same sums in the same order as on the wider tiles, so the
    outputs must be identical bit for bit, and meet the oracle."""
    p = O.make_block_params(D, E, 2, ratio, n_shared, seed=51, dtype=dtype, variant=variant)
    if variant == "gelu_tanh":
        _bias_params(p, 52, dtype)
    x = torch.randn(1, N, D, generator=_gen(53)).to(dtype)
    blk = block_from_params(p, D, variant, dtype, dev)
    slim, wide = _slim_and_not(blk, x.to(dev))
    want, _, _, logits = O.sparse_moe_block_forward(p, x)
    ok = ~O.gate_tie_rows(logits, 2).view(-1)
    tol = BF16_TOL if dtype == torch.bfloat16 else F16_TOL
    check_rows(slim.view(-1, D)[ok], want.view(-1, D)[ok], tol, "128-row tiles vs oracle")
    # (biased launches whose other choice is the 256-row tile, which starts its sums from the bias, never take
    # them: the parameter with D = 768 checks that the hook leaves those alone)
    assert torch.equal(slim, wide), "128-row weight tiles changed the result"
    # (and the default choice is one of the two)
    dflt = blk(x.to(dev)).cpu()
    assert torch.equal(dflt, wide) or torch.equal(dflt, slim)


@pytest.mark.parametrize("D,ratio,E,n_shared,N,dtype", [
    (1152, 4, 8, 2, 256, torch.bfloat16),     # one image: what the model picks them for
    (1152, 4, 8, 2, 77, torch.bfloat16),      # ragged, most tiles hold a handful of rows
    (1152, 4, 8, 2, 1000, torch.bfloat16),    # (hook only: the model leaves this size alone)
    (768, 2, 4, 2, 640, torch.float16),       # the fp16 build
    (1024, 2, 16, 0, 512, torch.bfloat16),    # no shared expert: one problem per launch
])
def test_fc1_on_128_row_weight_tiles(dev, D, ratio, E, n_shared, N, dtype):
    """SwiGLU fc1 with gathered rows on 128 weight rows per tile (64 gate + 64 up: the kernel
    with the generated k-loop, wave tile 128 x 64 with one output block per wave): the same
    sums in the same order as on the 256-row tiles, so the outputs must be identical bit for
    bit, and meet the oracle."""
    from dice_amd import lib
    p = O.make_block_params(D, E, 2, ratio, n_shared, seed=61, dtype=dtype, variant="swiglu")
    x = torch.randn(1, N, D, generator=_gen(63)).to(dtype)
    blk = block_from_params(p, D, "swiglu", dtype, dev)
    try:
        lib.load().dice_set_gemm_config(54, 0)
        slim = blk(x.to(dev)).clone().cpu()
        lib.load().dice_set_gemm_config(55, 0)
        wide = blk(x.to(dev)).clone().cpu()
    finally:
        lib.load().dice_set_gemm_config(0, 0)
    want, _, _, logits = O.sparse_moe_block_forward(p, x)
    ok = ~O.gate_tie_rows(logits, 2).view(-1)
    tol = BF16_TOL if dtype == torch.bfloat16 else F16_TOL
    check_rows(slim.view(-1, D)[ok], want.view(-1, D)[ok], tol, "128-row fc1 tiles vs oracle")
    assert torch.equal(slim, wide), "128-row weight tiles changed the result"
    dflt = blk(x.to(dev)).cpu()
    assert torch.equal(dflt, wide)
