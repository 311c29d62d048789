"""GPU parity of the fused caller: LayerNorm + adaLN modulation in front of the
layer and the gated residual behind it (the MoE line of DiTBlock.forward)."""
import pytest
import torch

from oracle import dice_oracle as O
from tests.helpers import block_from_params, rel_l2

pytestmark = pytest.mark.gpu

FP32_TOL = 1e-4
BF16_TOL = 2e-2


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from dice_amd import lib
    lib.load()
    return torch.device("cuda:0")


def _gen(seed):
    return torch.Generator().manual_seed(seed)


def _inputs(B, T, D, dtype, seed):
    g = _gen(seed)
    x = (torch.randn(B, T, D, generator=g) * 2 + 0.5).to(dtype)      # off-centre rows: the mean matters
    shift, scale, gate = ((torch.randn(B, D, generator=g) * 0.3).to(dtype) for _ in range(3))
    return x, shift, scale, gate


@pytest.mark.parametrize("B,T,D,dtype", [
    (3, 37, 384, torch.float32),      # ragged token count, one chunk round per lane
    (2, 256, 1152, torch.bfloat16),   # DiT-XL width: 144 chunks -> three rounds, the last partial
    (1, 5, 2048, torch.bfloat16),
    (2, 16, 64, torch.float16),
    (1, 3, 4096, torch.float32),      # sixteen rounds
])
def test_ln_modulate_matches_oracle(dev, B, T, D, dtype):
    from dice_amd import ops
    x, shift, scale, _ = _inputs(B, T, D, dtype, 3)
    want = O.norm_modulate(x, shift, scale, single_rounding=True)
    got = ops.ln_modulate(x.to(dev), shift.to(dev), scale.to(dev)).cpu()
    if dtype == torch.float32:
        assert torch.allclose(got, want, atol=2e-5, rtol=1e-5)
    else:
        # one rounding on both sides: at most one unit in the last place apart
        ulp = 2.0 ** (-7 if dtype == torch.bfloat16 else -10)   # upper end of a binade's relative spacing
        assert ((got.float() - want.float()).abs() <= ulp * want.float().abs().clamp_min(1e-3) * 1.01).all()
        assert (got != want).float().mean() < 0.02
    # and close to the literal four-rounding sequence of the reference module
    assert rel_l2(got, O.norm_modulate(x, shift, scale)) < (FP32_TOL if dtype == torch.float32 else BF16_TOL)


def test_combine_residual_matches_definition(dev):
    from dice_amd.lib import check, dtype_code, load, ptr, stream_ptr
    g = _gen(5)
    B, T, D, k = 2, 33, 128, 2
    N = B * T
    slot = torch.randn(N * k, D, generator=g)
    w = torch.rand(N, k, generator=g)
    shared = torch.randn(N, D, generator=g)
    resid = torch.randn(N, D, generator=g)
    gate = torch.randn(B, D, generator=g)
    want = resid.double() + gate.double().repeat_interleave(T, 0) * (
        (slot.double().view(N, k, D) * w.double()[:, :, None]).sum(1) + shared.double())
    d = [t.to(dev) for t in (slot, w, shared, resid, gate)]
    out = torch.empty(N, D, device=dev)
    check(load().dice_combine_residual(ptr(d[0]), None, ptr(d[1]), ptr(d[2]), None, None, None, ptr(d[3]),
                                       ptr(d[4]), T, ptr(out), dtype_code(torch.float32), N, k, D,
                                       stream_ptr()))
    assert torch.allclose(out.cpu().double(), want, atol=1e-5)
    # in place on the residual stream
    check(load().dice_combine_residual(ptr(d[0]), None, ptr(d[1]), ptr(d[2]), None, None, None, ptr(d[3]),
                                       ptr(d[4]), T, ptr(d[3]), dtype_code(torch.float32), N, k, D,
                                       stream_ptr()))
    assert torch.equal(d[3], out)


@pytest.mark.parametrize("variant", ["swiglu", "gelu_tanh"])
def test_block_half_fp32(dev, variant):
    """C1 shape in fp32: routing exact away from near-ties (the fused
    LayerNorm's last-bit differences move logits by ~1e-6), output at 1e-4."""
    B, T, D = 4, 256, 384
    p = O.make_block_params(D, 8, 2, 4, 2, seed=0, variant=variant)
    x, shift, scale, gate = _inputs(B, T, D, torch.float32, 7)
    want, h, widx, _, logits = O.dit_block_moe_half(p, x, shift, scale, gate)
    blk = block_from_params(p, D, variant, torch.float32, dev)
    got = blk.forward_modulated(x.to(dev), shift.to(dev), scale.to(dev), gate.to(dev)).cpu()
    ok = ~O.gate_tie_rows(logits, 2, tol=1e-4).view(B, T)
    assert ok.float().mean() > 0.99
    assert rel_l2(got[ok], want[ok]) < FP32_TOL
    # the two-step path (prologue op, plain layer, torch epilogue) agrees with the fused call
    from dice_amd import ops
    hd = ops.ln_modulate(x.to(dev), shift.to(dev), scale.to(dev))
    two = (x.to(dev) + gate.to(dev).unsqueeze(1) * blk(hd)).cpu()
    assert rel_l2(got, two) < 1e-6
    idx = torch.empty(B * T, 2, dtype=torch.int32, device=dev)
    blk.run(hd.view(-1, D), topk_idx_out=idx)
    assert torch.equal(idx.cpu().long()[ok.view(-1)], widx[ok.view(-1)])


def test_block_half_bf16_full_size(dev):
    """C2 shape, bf16, B = 32 samples of 256 tokens.  Checked against the
    oracle evaluated with the fused pass's precision (fp32 prologue and
    epilogue, one rounding each): routing exact away from ties, 2e-2 on the
    stream update; and against the literal four-rounding sequence on the rows
    where both route alike."""
    B, T, D = 32, 256, 1152
    p = O.make_block_params(D, 8, 2, 4, 2, seed=1, dtype=torch.bfloat16)
    x, shift, scale, gate = _inputs(B, T, D, torch.bfloat16, 9)
    blk = block_from_params(p, D, "swiglu", torch.bfloat16, dev)
    xd = x.to(dev)
    got = blk.forward_modulated(xd, shift.to(dev), scale.to(dev), gate.to(dev)).cpu()
    # in place on the stream gives the same bits
    x2 = xd.clone()
    blk.forward_modulated(x2, shift.to(dev), scale.to(dev), gate.to(dev), out=x2)
    assert torch.equal(x2.cpu(), got)
    sub = torch.arange(0, B * T, 16)                    # every 16th token: the CPU oracle in bf16 is slow
    sb = sub // T
    xs = x.view(-1, D)[sub].unsqueeze(1)                # [n, 1, D]: one token per "sample"
    want, h, widx, _, logits = O.dit_block_moe_half(p, xs, shift[sb], scale[sb], gate[sb], single_rounding=True)
    # The layer input the GPU routed on differs from the oracle's by one bf16 ulp in ~1 % of
    # its elements (tested above), which moves logits by ~1e-3: rows the GPU routed otherwise
    # must be few and must all have a routing margin of that order; they are set aside.
    from dice_amd import ops
    hd = ops.ln_modulate(xd, shift.to(dev), scale.to(dev))
    gidx = torch.empty(B * T, 2, dtype=torch.int32, device=dev)
    blk.run(hd.view(-1, D), topk_idx_out=gidx)
    gidx = gidx.cpu().long()[sub]
    moved = (gidx != widx).any(-1)
    assert moved.float().mean() < 0.01
    assert O.gate_tie_rows(logits, 2, tol=2e-2)[moved].all()
    ok = ~moved
    gs = got.view(-1, D)[sub]
    assert rel_l2(gs[ok], want[:, 0][ok]) < BF16_TOL
    # the update alone (the stream's own rounding is a large part of its error)
    assert rel_l2((gs.float() - xs[:, 0].float())[ok], (want[:, 0].float() - xs[:, 0].float())[ok]) < 6e-2
    # against the literal four-rounding op sequence, on the rows where both route alike
    lit, _, lidx, _, _ = O.dit_block_moe_half(p, xs, shift[sb], scale[sb], gate[sb])
    same = ok & (lidx == widx).all(-1)
    assert same.float().mean() > 0.9
    assert rel_l2(gs[same], lit[:, 0][same]) < BF16_TOL


def test_block_half_lagged_writes_entry_in_place(dev):
    """Displaced mode with the fused caller: the modulated rows go straight into
    the cached entry, and the results follow the oracle's state machine run on
    the oracle's own modulated inputs."""
    from dice_amd import ParaMode, diep
    B, T, D = 2, 96, 256
    p = O.make_block_params(D, 8, 2, 4, 2, seed=3, gate_std=0.1)
    pm = ParaMode(ep=True, ep_async=True, ep_async_mode="all")
    blk = block_from_params(p, D, "swiglu", torch.float32, dev, para_mode=pm)
    diep.ep_cache_init(cache_capacity=1)
    diep.use_latest_expert_weights(True)
    state = O.DiepState(1, use_latest_expert_weights=True)
    g = _gen(13)
    try:
        for t in range(4):
            x, shift, scale, gate = _inputs(B, T, D, torch.float32, 20 + t)
            if t == 0:
                diep.diep_force_sync()
                diep.ep_cache_clear()
                state.force_sync()
                state.cache_clear()
            want, *_ = O.dit_block_moe_half(p, x, shift, scale, gate, state=state, async_op=True, cache_key=0)
            got = blk.forward_modulated(x.to(dev), shift.to(dev), scale.to(dev), gate.to(dev)).cpu()
            if t == 0:
                diep.diep_cancel_sync()
                state.cancel_sync()
            assert rel_l2(got, want) < FP32_TOL, f"step {t}"
    finally:
        diep.ep_cache_init(cache_capacity=1)
        diep.use_latest_expert_weights(False)
        if diep.diep_forced_sync():
            diep.diep_cancel_sync()


def test_block_half_f16(dev):
    """The fused caller in fp16 (model.half() in the reference) at XL width."""
    B, T, D = 4, 256, 1152
    p = O.make_block_params(D, 8, 2, 4, 2, seed=2, dtype=torch.float16)
    x, shift, scale, gate = _inputs(B, T, D, torch.float16, 15)
    blk = block_from_params(p, D, "swiglu", torch.float16, dev)
    got = blk.forward_modulated(x.to(dev), shift.to(dev), scale.to(dev), gate.to(dev)).cpu()
    want, h, widx, _, logits = O.dit_block_moe_half(p, x, shift, scale, gate, single_rounding=True)
    from dice_amd import ops
    hd = ops.ln_modulate(x.to(dev), shift.to(dev), scale.to(dev))
    gidx = torch.empty(B * T, 2, dtype=torch.int32, device=dev)
    blk.run(hd.view(-1, D), topk_idx_out=gidx)
    moved = (gidx.cpu().long() != widx).any(-1)
    assert moved.float().mean() < 0.01
    ok = ~moved.view(B, T)
    assert rel_l2(got[ok], want[ok]) < 4e-3


def test_half_model_under_autocast_with_fp32_stream(dev):
    """The reference's serving set-up for XL / G (sample_ddp.py:97-98,228): the
    model in fp16, activations arriving in fp32 under torch.autocast.  The
    block casts like autocast's linear layers do and answers in fp16; the fused
    caller keeps an fp32 residual stream in fp32."""
    from dice_amd import DiceError
    B, T, D = 2, 128, 1152
    p = O.make_block_params(D, 8, 2, 4, 2, seed=4, dtype=torch.float16)
    blk = block_from_params(p, D, "swiglu", torch.float16, dev)
    x, shift, scale, gate = _inputs(B, T, D, torch.float32, 17)
    with pytest.raises(DiceError, match="autocast"):
        blk(x.to(dev))
    with torch.autocast(device_type="cuda", dtype=torch.float16):
        y = blk(x.to(dev))
        out = blk.forward_modulated(x.to(dev), shift.to(dev), scale.to(dev), gate.to(dev))
    assert y.dtype == torch.float16 and out.dtype == torch.float32
    want_y, _, _, logits = O.sparse_moe_block_forward(p, x.half())
    ok = ~O.gate_tie_rows(logits, 2).view(B, T)
    assert rel_l2(y.cpu()[ok], want_y[ok]) < 4e-3
    h = O.norm_modulate(x, shift, scale)
    wy, _, _, logits2 = O.sparse_moe_block_forward(p, h.half())
    want = x + gate.unsqueeze(1) * wy.float()
    ok2 = ~O.gate_tie_rows(logits2, 2, tol=1e-3).view(B, T)
    assert rel_l2(out.cpu()[ok2], want[ok2]) < 4e-3


def test_strided_adaln_chunks(dev):
    """shift / scale / gate as the reference hands them over: chunks of ONE
    adaLN output tensor (``self.adaLN_modulation(c).chunk(6, dim=1)``,
    models.py:515), i.e. strided views.  Every wrapper must keep its contiguous
    copies alive until the launch; a copy freed early is overwritten by the
    next one (shift and scale would then read the same memory)."""
    from dice_amd import ops
    B, T, D = 3, 64, 384
    g = _gen(23)
    x = (torch.randn(B, T, D, generator=g) * 2 + 0.5)
    c = torch.randn(B, 6 * D, generator=g) * 0.3
    cd = c.to(dev)
    shift_msa, scale_msa, gate_msa, shift, scale, gate = cd.chunk(6, dim=1)
    assert not shift.is_contiguous() and not scale.is_contiguous()
    w_shift, w_scale, w_gate = c.chunk(6, dim=1)[3:]
    want = O.norm_modulate(x, w_shift, w_scale, single_rounding=True)
    got = ops.ln_modulate(x.to(dev), shift, scale).cpu()
    assert torch.allclose(got, want, atol=2e-5, rtol=1e-5)
    # the whole line, same-dtype branch (fused prologue / epilogue)
    p = O.make_block_params(D, 8, 2, 4, 2, seed=5, gate_std=0.1)
    blk = block_from_params(p, D, "swiglu", torch.float32, dev)
    want_line, _, _, _, logits = O.dit_block_moe_half(p, x, w_shift, w_scale, w_gate, single_rounding=True)
    ok = ~O.gate_tie_rows(logits, 2, tol=1e-4).view(B, T)
    out = blk.forward_modulated(x.to(dev), shift, scale, gate).cpu()
    assert rel_l2(out[ok], want_line[ok]) < FP32_TOL
    # mixed-precision branch: fp16 block under autocast, fp32 stream and fp32 strided chunks
    p16 = O.make_block_params(D, 8, 2, 4, 2, seed=5, gate_std=0.1, dtype=torch.float16)
    blk16 = block_from_params(p16, D, "swiglu", torch.float16, dev)
    with torch.autocast(device_type="cuda", dtype=torch.float16):
        out16 = blk16.forward_modulated(x.to(dev), shift, scale, gate).cpu()
    h = O.norm_modulate(x, w_shift, w_scale)
    wy, _, _, logits2 = O.sparse_moe_block_forward(p16, h.half())
    want16 = x + w_gate.unsqueeze(1) * wy.float()
    ok2 = ~O.gate_tie_rows(logits2, 2, tol=1e-3).view(B, T)
    assert rel_l2(out16[ok2], want16[ok2]) < 4e-3
    with pytest.raises(Exception, match="shift and scale"):
        ops.ln_modulate(x.to(dev), shift[:, :-8], scale)


def test_stale_mask_or_cache_is_refused_before_launch(dev):
    """A skip mask or cache tensor left over from another batch size would be
    indexed out of bounds by the kernels; the host side raises instead (the
    reference fails with a shape error in the same situation).  Nothing is
    launched on the refused calls."""
    from dice_amd import DiceError, diep, ops
    from dice_amd.lib import MODE_PUT, MODE_SKIP
    D, E, N = 256, 8, 256
    p = O.make_block_params(D, E, 2, 4, 2, seed=6)
    blk = block_from_params(p, D, "swiglu", torch.float32, dev, ep=True, layer_idx=0)
    x = torch.randn(N, D, generator=_gen(6)).to(dev)
    mask = O.skip_mask(2 * N, "high").to(dev)
    cache = torch.empty_like(x)
    blk.run(x, MODE_PUT, mask, None, cache)
    with pytest.raises(DiceError, match="skip mask"):
        blk.run(x, MODE_SKIP, mask[:-2], cache, None)
    with pytest.raises(DiceError, match="skip mask"):
        blk.run(x, MODE_SKIP, mask.cpu(), cache, None)
    with pytest.raises(DiceError, match="cache_in"):
        blk.run(x, MODE_SKIP, mask, cache[: N // 2], None)
    with pytest.raises(DiceError, match="cache_in"):
        blk.run(x, MODE_SKIP, mask, cache.half(), None)
    with pytest.raises(DiceError, match="cache_out"):
        blk.run(x, MODE_PUT, mask, None, torch.empty(N, D // 2, device=dev))
    with pytest.raises(DiceError, match="needs cache_in"):
        blk.run(x, MODE_SKIP, mask, None, None)
    # through the module: the batch grows between a full step and the skip step that follows
    diep.ep_cache_init(cache_capacity=1, noskip_step=2, skip_mode="rand")
    diep.ep_set_rand_mask(None)
    try:
        diep.ep_set_step(8)
        diep.ep_cache_clear()
        blk(x.view(1, N, D))
        diep.ep_set_step(7)
        assert diep.ep_skip_now(0)
        with pytest.raises(DiceError, match="rand"):
            blk(torch.cat([x, x]).view(1, 2 * N, D))      # the 'rand' mask was drawn for N tokens
        diep.ep_cache_init(cache_capacity=1, noskip_step=2, skip_mode="high")
        diep.ep_set_step(8)
        blk(x.view(1, N, D))
        diep.ep_set_step(7)
        with pytest.raises(DiceError, match="cache_in"):
            blk(torch.cat([x, x]).view(1, 2 * N, D))      # cached rows of N tokens, 2N arrive
    finally:
        diep.ep_cache_init(cache_capacity=1, noskip_step=1)
    # caller-supplied routing with an expert id outside the table: the slot is dropped and adds nothing
    idx = torch.randint(0, E, (2 * N,), generator=_gen(7))
    w = torch.rand(2 * N, 1, generator=_gen(8))
    bad = idx.clone()
    bad[5], bad[100] = E, -1
    y_bad = blk.moe_infer(x, bad.to(dev), w.to(dev)).cpu()
    w0 = w.clone()
    w0[5], w0[100] = 0, 0
    y_ref = blk.moe_infer(x, idx.to(dev), w0.to(dev)).cpu()
    assert torch.allclose(y_bad, y_ref, atol=1e-6)
    torch.cuda.synchronize()
