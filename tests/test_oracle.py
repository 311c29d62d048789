"""Pins the CPU oracle: golden fixtures, closed forms, invariants, brute force.

None of these tests retype an oracle formula in torch; each compares against a
float64 numpy definition, a fixture computed without the oracle, or a property
the mathematics fixes.
"""
import os

import numpy as np
import pytest
import torch

from oracle import dice_oracle as O


class LinearExpert:
    def __init__(self, w, b):
        self.w, self.b = torch.from_numpy(w), torch.from_numpy(b)

    def __call__(self, x):
        return torch.nn.functional.linear(x, self.w, self.b)


@pytest.mark.parametrize("seed", [42, 43])
def test_moe_infer_matches_reference_recipe(golden_dir, seed):
    """tests/test_ep.py's recipe: single-node and EP data flows agree with the
    per-token float64 definition within the reference's own tolerance."""
    z = np.load(os.path.join(golden_dir, f"ep_recipe_seed{seed}.npz"))
    experts = [LinearExpert(z["expert_w"][e], z["expert_b"][e]) for e in range(8)]
    for it in range(4):
        x = torch.from_numpy(z[f"inp{it}"])
        idx = torch.from_numpy(z[f"idx{it}"])
        w = torch.from_numpy(z[f"w{it}"])
        want = torch.from_numpy(z[f"y{it}"]).float()
        got = O.moe_infer(x, experts, idx, w, 2)
        got_ep = O.moe_infer_ep_local(x, experts, idx, w, 2)
        assert torch.allclose(got, want, atol=1e-6, rtol=1e-5)
        assert torch.allclose(got_ep, want, atol=1e-6, rtol=1e-5)
        assert torch.allclose(got_ep, got, atol=1e-6)


def test_gate_against_bruteforce_fixture(golden_dir):
    z = np.load(os.path.join(golden_dir, "gate_small.npz"))
    idx, w, logits = O.gate_forward(torch.from_numpy(z["x"]), torch.from_numpy(z["w"]), 2)
    assert torch.equal(idx, torch.from_numpy(z["idx"]))
    np.testing.assert_allclose(w.numpy(), z["weight"], rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(logits.numpy(), z["logits"], rtol=1e-5, atol=1e-6)
    _, wn, _ = O.gate_forward(torch.from_numpy(z["x"]), torch.from_numpy(z["w"]), 2, norm_topk_prob=True)
    np.testing.assert_allclose(wn.numpy(), z["weight_norm"], rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("E,k", [(8, 2), (16, 2), (16, 4), (5, 3)])
def test_gate_invariants(E, k):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(301, 64, generator=g)
    w = torch.randn(E, 64, generator=g) * 0.2
    idx, wt, logits = O.gate_forward(x, w, k)
    assert idx.dtype == torch.int64 and idx.shape == (301, k)
    assert (wt[:, :-1] >= wt[:, 1:]).all(), "slot order must be descending score"
    assert all(len(set(r.tolist())) == k for r in idx), "experts of a token are distinct"
    assert (wt.sum(-1) <= 1 + 1e-6).all() and (wt > 0).all()
    # slot 0 is the arg-max of the logits; the top-k set equals numpy's.
    assert torch.equal(idx[:, 0], logits.argmax(-1))
    want = np.argsort(-logits.double().numpy(), axis=-1, kind="stable")[:, :k]
    assert np.array_equal(np.sort(idx.numpy(), -1), np.sort(want, -1))
    _, wn, _ = O.gate_forward(x, w, k, norm_topk_prob=True)
    assert torch.allclose(wn.sum(-1), torch.ones(301), atol=1e-6)
    # bias extension shifts logits
    b = torch.randn(E, generator=g)
    _, _, lb = O.gate_forward(x, w, k, bias=b)
    assert torch.allclose(lb, logits + b, atol=1e-6)


def test_gate_bf16_inputs_use_fp32_arithmetic():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(64, 128, generator=g).bfloat16()
    w = (torch.randn(8, 128, generator=g) * 0.02).bfloat16()
    _, _, logits = O.gate_forward(x, w, 2)
    ref = x.double() @ w.double().T
    assert logits.dtype == torch.float32
    assert torch.allclose(logits.double(), ref, atol=1e-6)


def test_tie_rows_flags_small_gaps():
    logits = torch.tensor([[3.0, 2.0, 1.0, 0.0], [3.0, 3.0 - 5e-7, 1.0, 0.0], [3.0, 2.0, 2.0, 0.0],
                           [3.0, 2.0, 1.0, 1.0]])
    assert O.gate_tie_rows(logits, 2).tolist() == [False, True, True, False]


def _np_silu(v):
    return v / (1.0 + np.exp(-v))


@pytest.mark.parametrize("tp", [1, 2])
def test_swiglu_closed_form(tp):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((19, 32))
    wg, wu = rng.standard_normal((64, 32)) * 0.2, rng.standard_normal((64, 32)) * 0.2
    wd = rng.standard_normal((32, 64)) * 0.2
    want = (_np_silu(x @ wg.T) * (x @ wu.T)) @ wd.T
    got = O.moe_mlp(*(torch.from_numpy(a).float() for a in (x, wg, wu, wd)), pretraining_tp=tp)
    np.testing.assert_allclose(got.numpy(), want, rtol=1e-4, atol=1e-5)
    # a transposed down_proj or swapped gate/up must not pass
    swapped = O.moe_mlp(*(torch.from_numpy(a).float() for a in (x, wu, wg, wd)), pretraining_tp=tp)
    assert not np.allclose(swapped.numpy(), want, rtol=1e-2, atol=1e-3)


def test_gelu_closed_form():
    rng = np.random.default_rng(4)
    x = rng.standard_normal((11, 16))
    w1, b1 = rng.standard_normal((48, 16)) * 0.3, rng.standard_normal(48) * 0.1
    w2, b2 = rng.standard_normal((16, 48)) * 0.3, rng.standard_normal(16) * 0.1
    a = x @ w1.T + b1
    gelu = 0.5 * a * (1 + np.tanh(np.sqrt(2 / np.pi) * (a + 0.044715 * a ** 3)))
    want = gelu @ w2.T + b2
    got = O.gelu_mlp(*(torch.from_numpy(v).float() for v in (x, w1, b1, w2, b2)))
    np.testing.assert_allclose(got.numpy(), want, rtol=1e-4, atol=1e-5)


def test_dispatch_tables_invariants():
    g = torch.Generator().manual_seed(5)
    idx = torch.randint(0, 8, (2048,), generator=g)
    idx[idx == 3] = 4  # an empty expert
    counts, offsets, perm, inv = O.dispatch_tables(idx, 8)
    assert counts.tolist() == np.bincount(idx.numpy(), minlength=8).tolist()
    assert counts[3] == 0
    assert offsets.tolist() == [0] + np.cumsum(counts.numpy()).tolist()
    assert sorted(perm.tolist()) == list(range(2048))
    grouped = idx[perm]
    assert (grouped[1:] >= grouped[:-1]).all()
    assert torch.equal(inv[perm], torch.arange(2048))
    for e in range(8):
        seg = perm[offsets[e]:offsets[e + 1]]
        assert (seg[1:] > seg[:-1]).all(), "stable: ascending slot inside a group"
    # group membership equals the reference's unstable argsort
    ref = idx.argsort()
    for e in range(8):
        assert set(ref[offsets[e]:offsets[e + 1]].tolist()) == set(perm[offsets[e]:offsets[e + 1]].tolist())


def _small_block(dtype=torch.float32, variant="swiglu", seed=0, E=8, D=64):
    return O.make_block_params(D, E, top_k=2, mlp_ratio=2, n_shared=2, seed=seed, dtype=dtype,
                               variant=variant, gate_std=0.5)


@pytest.mark.parametrize("variant", ["swiglu", "gelu_tanh"])
def test_block_equals_dense_definition(variant):
    p = _small_block(variant=variant)
    x = torch.randn(2, 24, 64, generator=torch.Generator().manual_seed(6))
    y, idx, wt, _ = O.sparse_moe_block_forward(p, x)
    y_ep, _, _, _ = O.sparse_moe_block_forward(p, x, use_ep_path=True)
    dense = O.dense_moe(x.view(-1, 64), p.experts, idx, wt) + p.shared(x.view(-1, 64))
    assert torch.allclose(y.view(-1, 64), dense, atol=1e-5)
    assert torch.allclose(y_ep, y, atol=1e-5)


def test_skip_identities():
    """(i) a skip step that blends with THIS step's own unscaled outputs equals
    the full step; (ii) closed form of the blend with a foreign cache;
    (iii) 'high' and 'low' exchange roles when the two slots are swapped."""
    p = _small_block(seed=9)
    g = torch.Generator().manual_seed(10)
    x = torch.randn(40, 64, generator=g)
    idx, wt, _ = O.gate_forward(x, p.gate_weight, 2)
    flat_idx, flat_w = idx.reshape(-1), wt.reshape(-1, 1)
    full = O.moe_infer_ep_local(x, p.experts, flat_idx, flat_w, 2)
    for mode in ("high", "low", "rand"):
        mask = O.skip_mask(80, mode)
        assert mask.view(40, 2).sum(1).eq(1).all()
        cache = O.EPSkipCache(1)
        put = O.moe_infer_ep_local(x, p.experts, flat_idx, flat_w, 2, mask, False, cache, 0)
        assert torch.allclose(put, full, atol=1e-6), "a put step returns the full result"
        assert cache.contains(0) and cache.cache[0].shape == (40, 64)
        skipped = O.moe_infer_ep_local(x, p.experts, flat_idx, flat_w, 2, mask, True, cache, 0)
        assert torch.allclose(skipped, full, atol=1e-5)
        assert not cache.contains(0), "get empties the entry"
        # foreign cache: closed form per token
        C = torch.randn(40, 64, generator=g)
        cache.put(0, C)
        got = O.moe_infer_ep_local(x, p.experts, flat_idx, flat_w, 2, mask, True, cache, 0)
        m2 = mask.view(40, 2)
        for t in range(40):
            s = int(m2[t].nonzero()[0])
            r = 1 - s
            want = wt[t, s] * C[t] + wt[t, r] * p.experts[int(idx[t, r])](x[t:t + 1])[0]
            assert torch.allclose(got[t], want, atol=1e-5)
    # slot swap symmetry
    C = torch.randn(40, 64, generator=g)
    sw_idx, sw_w = idx.flip(1).reshape(-1), wt.flip(1).reshape(-1, 1)
    c1, c2 = O.EPSkipCache(1), O.EPSkipCache(1)
    c1.put(0, C)
    c2.put(0, C)
    a = O.moe_infer_ep_local(x, p.experts, flat_idx, flat_w, 2, O.skip_mask(80, "high"), True, c1, 0)
    b = O.moe_infer_ep_local(x, p.experts, sw_idx, sw_w, 2, O.skip_mask(80, "low"), True, c2, 0)
    assert torch.allclose(a, b, atol=1e-6)


def test_skip_schedule_interval_two():
    """Reference schedule (rectified_flow.py:83-105, diep.py:61-68): steps count
    down 50..1, the first is full, then odd steps skip and even steps are full."""
    cache = O.EPSkipCache(1)
    pattern = []
    for i in range(50, 0, -1):
        if i == 50:
            cache.clear()
        now = O.skip_now(True, cache, 0, i, 2)
        pattern.append(now)
        if now:
            assert cache.get(0) is not None
        else:
            cache.put(0, torch.zeros(1))
    assert pattern[0] is False
    assert pattern[1:] == [(i % 2 != 0) for i in range(49, 0, -1)]
    assert not any(a and b for a, b in zip(pattern, pattern[1:])), "never two skips in a row"


def test_fp8_rowwise_quantiser_properties():
    g = torch.Generator().manual_seed(11)
    w = O.xavier_uniform(96, 64, g)
    w[5] = 0
    q, s = O.quantize_fp8_rowwise(w)
    assert q.dtype == torch.float8_e4m3fn and s.shape == (96,)
    assert s[5] == 1.0 and (q[5].float() == 0).all()
    deq = O.dequantize_fp8_rowwise(q, s)
    amax = w.abs().amax(1)
    # the row maximum maps to +-448 exactly; e4m3 keeps 3 mantissa bits
    assert torch.allclose(deq.abs().amax(1)[amax > 0], amax[amax > 0], rtol=1e-6)
    rel = (deq - w).abs() / amax[:, None].clamp_min(1e-30)
    assert rel.max() <= 2 ** -4 + 1e-6
    big = w.abs() > amax[:, None] / 16
    assert ((deq - w).abs()[big] <= w.abs()[big] * 2 ** -4 + 1e-9).all()


def _e4m3_codes():
    """The 127 non-negative finite e4m3fn values by their bit pattern (float64)."""
    c = np.arange(127)
    e, m = c >> 3, c & 7
    return np.where(e == 0, m * 2.0 ** -9, (1 + m / 8.0) * 2.0 ** (e.astype(np.float64) - 7))


def _nearest_e4m3(p):
    """Nearest code of every element of p (float64 magnitudes within 448), ties
    to the even bit pattern: brute force over all codes."""
    vals = _e4m3_codes()
    d = np.abs(np.abs(p)[..., None] - vals)
    best = d.argmin(-1)                               # first minimum = the lower code
    nxt = np.minimum(best + 1, 126)
    tie = (np.take_along_axis(d, nxt[..., None], -1)[..., 0] == d.min(-1)) & (nxt != best)
    best = np.where(tie & (best % 2 == 1), nxt, best)
    return (best | np.where(np.signbit(p), 128, 0)).astype(np.uint8)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fp8_act_quantiser_against_bruteforce(dtype):
    """Bytes of ``quantize_fp8_act`` against a search over all e4m3 codes in
    numpy (float32 quotient 448 / amax by IEEE division, float32 product, then
    the nearest code, ties to even).  16-bit inputs are often simple fractions of
    the row maximum, which puts products within an ulp of a tie: there a quotient
    rounded twice (reciprocal times 448) picks the other code, and the last
    assertion checks that these rows hold such elements."""
    g = torch.Generator().manual_seed(384)
    x = (torch.randn(67, 384, generator=g) * torch.logspace(-3, 2, 67)[:, None]).to(dtype)
    x[3] = 0
    q, s = O.quantize_fp8_act(x)
    xn = x.float().numpy()
    amax = np.abs(xn).max(1)
    inv = np.where(amax > 0, np.float32(448.0) / np.where(amax > 0, amax, np.float32(1)), np.float32(1))
    prod = (xn * inv[:, None].astype(np.float32)).astype(np.float32)
    want = _nearest_e4m3(np.clip(prod.astype(np.float64), -448, 448))
    got = q.view(torch.uint8).numpy()
    zero = prod == 0                                  # the sign of a zero byte is not part of the contract
    assert np.array_equal(got[~zero], want[~zero]) and not (got[zero] & 0x7f).any()
    assert np.array_equal(s.numpy(), np.where(amax > 0, amax / np.float32(448.0), np.float32(1)).astype(np.float32))
    inv2 = (np.float32(1) / np.where(amax > 0, amax, np.float32(1))).astype(np.float32) * np.float32(448.0)
    prod2 = (xn * inv2[:, None].astype(np.float32)).astype(np.float32)
    twice = _nearest_e4m3(np.clip(prod2.astype(np.float64), -448, 448))
    assert (twice != want).any(), "no element near a tie: the data no longer tells the two quotients apart"


def test_fp8_act_quantiser_properties():
    g = torch.Generator().manual_seed(22)
    x = torch.randn(33, 128, generator=g).bfloat16()
    x[4] = 0
    q, s = O.quantize_fp8_act(x)
    assert q.dtype == torch.float8_e4m3fn and s.dtype == torch.float32 and s.shape == (33,)
    assert s[4] == 1.0 and (q[4].float() == 0).all()
    nz = torch.arange(33) != 4
    assert (q.float().abs().amax(1)[nz] == 448).all()                 # the row maximum maps to +-448
    # a power-of-two factor changes the scale by that factor and no byte
    q2, s2 = O.quantize_fp8_act((x.float() * 8).bfloat16())
    assert torch.equal(q2.view(torch.uint8), q.view(torch.uint8)) and torch.equal(s2[nz], s[nz] * 8)
    # idempotence: codes times a power-of-two scale re-quantise to the same codes
    y = (q.float() * 2.0 ** -5).bfloat16()                            # e4m3 values are exact in bf16
    q3, s3 = O.quantize_fp8_act(y)
    assert torch.equal(q3.view(torch.uint8)[nz], q.view(torch.uint8)[nz]) and (s3[nz] == 2.0 ** -5).all()
    deq = q.float() * s[:, None]
    assert ((deq - x.float()).abs() <= x.float().abs().amax(1, keepdim=True) * 2 ** -4).all()


def test_fp8_block_quantiser_against_bruteforce():
    """``quantize_fp8_act_blocks`` against its definition worked out another way: per block the
    exponent is the smallest e with amax * fp32(1/448) <= 2^(e-127) (found by a search over all 255
    exponents in float64, which holds every float32 and every power of two exactly), the bytes are the
    nearest e4m3 codes of block * 2^(127-e) (search over all codes, ties to even)."""
    g = torch.Generator().manual_seed(77)
    x = torch.randn(19, 256, generator=g) * torch.exp2(torch.randint(-30, 30, (19, 8), generator=g).float()
                                                       ).repeat_interleave(32, dim=1)
    x = x.bfloat16()
    x[2, 32:64] = 0
    x[5, 0:32] = 448.0 * 2.0 ** -7                    # amax / 448 a power of two: that very power
    x[6, 0:32] = 450.0 * 2.0 ** -7                    # just above it: the next power
    q, e = O.quantize_fp8_act_blocks(x)
    assert q.dtype == torch.float8_e4m3fn and e.dtype == torch.uint8 and e.shape == (19, 8)
    xn = x.float().numpy().reshape(19, 8, 32)
    amax = np.abs(xn).max(-1)
    t = (amax * np.float32(1.0 / 448.0)).astype(np.float32).astype(np.float64)
    pw = np.ldexp(1.0, np.arange(255) - 127)          # 2^(e-127), e = 0 .. 254
    want_e = (t[..., None] <= pw).argmax(-1)
    assert np.array_equal(e.numpy(), want_e)
    scaled = xn.astype(np.float64) * np.ldexp(1.0, 127 - want_e)[..., None]
    want_q = _nearest_e4m3(np.clip(scaled, -448, 448)).reshape(19, 256)
    got = q.view(torch.uint8).numpy()
    zero = scaled.reshape(19, 256) == 0
    assert np.array_equal(got[~zero], want_q[~zero]) and not (got[zero] & 0x7f).any()
    assert e[2, 1] == 0 and e[5, 0] == 127 - 7 and e[6, 0] == 127 - 6


def test_fp8_block_quantiser_properties():
    g = torch.Generator().manual_seed(23)
    x = torch.randn(33, 128, generator=g).bfloat16()
    q, e = O.quantize_fp8_act_blocks(x)
    deq = O.dequantize_fp8_act_blocks(q, e)
    blk_amax = x.float().view(33, 4, 32).abs().amax(-1)
    # the scaled block maximum lies in (224, 448] (the smallest power of two that keeps it representable),
    # so its code is one of 224 .. 448
    top = q.float().view(33, 4, 32).abs().amax(-1)
    assert (top >= 224).all() and (top <= 448).all()
    scaled = blk_amax * torch.exp2(127 - e.float())
    assert (scaled > 224).all() and (scaled <= 448).all()
    assert ((deq - x.float()).view(33, 4, 32).abs() <= blk_amax[..., None] * 2 ** -4).all()
    # a power-of-two factor per block moves the exponent by that power and changes no byte
    f = torch.tensor([3, -2, 0, 5]).repeat(33, 1)
    x2 = (x.float().view(33, 4, 32) * torch.exp2(f.float())[..., None]).reshape(33, 128).bfloat16()
    q2, e2 = O.quantize_fp8_act_blocks(x2)
    assert torch.equal(q2.view(torch.uint8), q.view(torch.uint8)) and torch.equal(e2.int(), e.int() + f)
    # idempotence of the values: what it returns re-quantises to the same numbers (a block whose maximum was
    # rounded down to the code 224 comes back with the next smaller exponent and doubled codes)
    q3, e3 = O.quantize_fp8_act_blocks(deq.bfloat16())       # e4m3 values times powers of two are exact in bf16
    assert torch.equal(O.dequantize_fp8_act_blocks(q3, e3), deq)
    assert ((e3 == e) | ((e3.int() == e.int() - 1) & (top == 224))).all()
    # blocks are independent; a block with an infinity or a NaN becomes NaN bytes with a unit scale
    y = x.clone()
    y[7, 40] = float("inf")
    y[8, 100] = float("nan")
    q4, e4 = O.quantize_fp8_act_blocks(y)
    same = torch.ones(33, 4, dtype=torch.bool)
    same[7, 1] = same[8, 3] = False
    assert torch.equal(q4.view(torch.uint8).view(33, 4, 32)[same], q.view(torch.uint8).view(33, 4, 32)[same])
    assert torch.equal(e4[same], e[same]) and e4[7, 1] == 127 and e4[8, 3] == 127
    assert (q4.view(torch.uint8).view(33, 4, 32)[~same] & 0x7f == 0x7f).all()
    assert torch.isnan(O.dequantize_fp8_act_blocks(q4, e4)[7, 32:64]).all()


def test_fp8_act_expert_with_h_blocks_is_the_product_of_dequantised_operands():
    p = O.make_block_params(256, 2, 1, 2, None, seed=5, dtype=torch.bfloat16)
    ex = O.Fp8ActExpert(p.experts[0], h_blocks=True)
    x = torch.randn(9, 256, generator=torch.Generator().manual_seed(6)).bfloat16()
    h = ex.hidden_act(x)
    assert torch.equal(h, O.Fp8ActExpert(p.experts[0]).hidden_act(x))      # fc1 is the same either way
    q, e = O.quantize_fp8_act_blocks(h)
    want = (O.dequantize_fp8_act_blocks(q, e).double() @ ex.q2.double().t()) * ex.s2.double()[None, :]
    got = ex(x).double()
    assert float((got - want).norm() / want.norm()) < 1e-2 and not torch.equal(ex(x), O.Fp8ActExpert(p.experts[0])(x))


@pytest.mark.parametrize("variant", ["swiglu", "gelu_tanh"])
def test_fp8_act_expert_is_the_product_of_dequantised_operands(variant):
    """``Fp8ActExpert`` against float64 numpy on the dequantised operands: the
    products of e4m3 codes are exact in float64, so only the rounding of ``h`` to
    bf16 (re-done here from the float64 value) and of the output differ."""
    D, I = 64, 128
    p = O.make_block_params(D, 2, 1, I // D, n_shared=0, seed=5, dtype=torch.bfloat16, variant=variant)
    ex = p.experts[0]
    if variant == "gelu_tanh":
        g = torch.Generator().manual_seed(6)
        ex.fc1_b = (torch.randn(I, generator=g) * 0.1).bfloat16()
        ex.fc2_b = (torch.randn(D, generator=g) * 0.1).bfloat16()
    x = torch.randn(48, D, generator=torch.Generator().manual_seed(7)).bfloat16()
    got_h = O.Fp8ActExpert(ex).hidden_act(x).float().numpy()
    got = O.Fp8ActExpert(ex)(x).float().numpy()

    def deq(t):
        q, s = O.quantize_fp8_act(t)
        return q.float().double().numpy() * s.double().numpy()[:, None]

    def wdeq(w):
        q, s = O.quantize_fp8_rowwise(w)
        return q.float().double().numpy() * s.double().numpy()[:, None]

    if variant == "swiglu":
        a = deq(x) @ wdeq(torch.cat([ex.gate_proj, ex.up_proj], 0)).T
        gate, up = a[:, :I], a[:, I:]
        h = gate / (1 + np.exp(-gate)) * up
        w2, b2 = ex.down_proj, 0.0
    else:
        a = deq(x) @ wdeq(ex.fc1_w).T + ex.fc1_b.double().numpy()
        h = 0.5 * a * (1 + np.tanh(np.sqrt(2 / np.pi) * (a + 0.044715 * a ** 3)))
        w2, b2 = ex.fc2_w, ex.fc2_b.double().numpy()
    assert np.abs(got_h - h).max() <= np.abs(h).max() * 2 ** -8
    # fc2 on the oracle's own h (its bf16 rounding is then shared)
    out = deq(torch.from_numpy(got_h).bfloat16()) @ wdeq(w2).T + b2
    assert np.abs(got - out).max() <= np.abs(out).max() * 2 ** -8


# --------------------------------------------------------------------------- #
# step-lagged expert parallelism (displaced / interweaved) on one worker
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("seed", [42, 43])
def test_displaced_lag_matches_reference_recipe(golden_dir, seed):
    """tests/test_ep.py:79-124 with async_op=True: iteration 0 is a forced-sync
    step, iteration 1 returns iteration 0's result and iteration t >= 2 returns
    iteration t-2's; expected values are the float64 per-token fixtures."""
    z = np.load(os.path.join(golden_dir, f"ep_recipe_seed{seed}.npz"))
    experts = [LinearExpert(z["expert_w"][e], z["expert_b"][e]) for e in range(8)]
    state = O.DiepState(1)
    for it in range(4):
        if it == 0:
            state.force_sync()
        elif it == 1:
            state.cancel_sync()
        x = torch.from_numpy(z[f"inp{it}"])
        idx = torch.from_numpy(z[f"idx{it}"])
        w = torch.from_numpy(z[f"w{it}"])
        got = O.moe_infer_ep_async(state, x, experts, idx, w, 2, True, cache_key=0)
        src = 0 if it < 2 else it - 2
        want = torch.from_numpy(z[f"y{src}"]).float()
        assert torch.allclose(got, want, atol=1e-6, rtol=1e-5), (it, src)


def _per_token(x, experts, idx, w, idx_for_experts=None):
    """float64 numpy definition y[t] = sum_j w[t,j] * E_{idx[t,j]}(x[t]) for
    LinearExpert lists."""
    x64 = x.double().numpy()
    n = x.shape[0]
    y = np.zeros((n, x.shape[1]))
    ids = idx if idx_for_experts is None else idx_for_experts
    for t in range(n):
        for j in range(2):
            e = experts[int(ids[2 * t + j])]
            y[t] += float(w[2 * t + j]) * (e.w.double().numpy() @ x64[t] + e.b.double().numpy())
    return torch.from_numpy(y).float()


def _rand_linear_experts(gen, n, d):
    return [LinearExpert(torch.rand(d, d, generator=gen).numpy(), torch.rand(d, generator=gen).numpy())
            for _ in range(n)]


@pytest.mark.parametrize("strategy", ["all", "shallow", "deep", "interleaved"])
@pytest.mark.parametrize("latest", [False, True])
def test_interweaved_lag_closed_form(strategy, latest):
    """Pipelined mode: a lagged layer returns its own previous-step result
    (own experts, own previous input, previous routing; the routing WEIGHTS are
    the current ones iff use_latest_expert_weights), layers outside the
    selective strategy stay exact, and a forced-sync step is exact everywhere."""
    L, n, d, E = 4, 24, 12, 4
    gen = torch.Generator().manual_seed(3)
    layers = [_rand_linear_experts(gen, E, d) for _ in range(L)]
    state = O.DiepState(L, async_pipeline=True, selective_async_strategy=strategy,
                        use_latest_expert_weights=latest)
    hist = []
    for step in range(4):
        forced = step == 0
        if forced:
            state.force_sync()
            state.cache_clear()
        cur = []
        for l in range(L):
            x = torch.randn(n, d, generator=gen)
            idx = torch.randint(0, E, (2 * n,), generator=gen)
            w = torch.rand(2 * n, 1, generator=gen)
            cur.append((x, idx, w))
            lagged = O.layer_is_async(strategy, l, L)
            got = O.moe_infer_ep_async(state, x, layers[l], idx, w, 2, lagged, cache_key=l)
            if forced or not lagged:
                want = _per_token(x, layers[l], idx, w)
            else:
                px, pidx, pw = hist[-1][l]
                want = _per_token(px, layers[l], pidx, w if latest else pw)
            assert torch.allclose(got, want, atol=1e-5, rtol=1e-5), (step, l)
        hist.append(cur)
        if forced:
            state.cancel_sync()


def _expert_row(experts, e, x64_row):
    ex = experts[int(e)]
    return ex.w.double().numpy() @ x64_row + ex.b.double().numpy()


@pytest.mark.parametrize("skip_mode", ["low", "high"])
@pytest.mark.parametrize("latest", [False, True])
@pytest.mark.parametrize("pipeline", [False, True])
def test_lag_with_skip_cache_closed_form(pipeline, latest, skip_mode):
    """Step lag together with conditional communication (interval 2) on the
    reference's countdown schedule, with a different input, routing and routing
    weights at every step and in every layer, against a float64 per-token
    definition that shares no code with the oracle (expertpara/ep_fwd.py:49-66,
    176-193; expertpara/diep.py:196-289; expertpara/ep_cache.py:215-220).

    What a call returns is fixed by three things.  (1) Which earlier call's
    routing and rows it emits: displaced mode emits step 0 at steps 0 and 1 and
    step t - 2 from then on; interweaved mode emits the layer's own step t - 1
    (step 0 at step 0).  (2) What kind of entry that was: a call made while
    ``ep_skip_now`` held dispatched only its unmasked slot, so its emission takes
    the masked slot's row from the skip cache (which ``get`` empties); a full
    entry's emission refills the cache with its masked slots' unweighted rows.
    (3) The routing weights: the emitting call's own when
    ``use_latest_expert_weights``, else those of the emitted entry.  A wrong lag
    (1 for 2), put and work swapped, a stale cache row or the wrong weights
    each change the result, because no two steps share an input here."""
    L, n, d, E, steps = (3 if pipeline else 1), 12, 8, 4, 9
    gen = torch.Generator().manual_seed(17 + int(pipeline))
    layers = [_rand_linear_experts(gen, E, d) for _ in range(L)]
    state = O.DiepState(L, noskip_step=2, skip_mode=skip_mode, async_pipeline=pipeline,
                        selective_async_strategy="all" if pipeline else None, use_latest_expert_weights=latest)
    mask = O.skip_mask(2 * n, skip_mode)
    m = 0 if skip_mode == "high" else 1          # the masked slot of every token; r = the other
    r = 1 - m
    hist = []                                    # per step, per layer: (x, idx, w, kind)
    cache_rows = [None] * L                      # the skip cache as this test keeps it: float64 rows [n, d] or None
    for t in range(steps):
        i = steps - t                            # the sampler counts down (rectified_flow.py:83-128)
        state.step = i
        forced = t == 0
        if forced:
            state.force_sync()
            state.cache_clear()
            cache_rows = [None] * L
        cur = []
        for l in range(L):
            x = torch.randn(n, d, generator=gen)
            idx = torch.stack([torch.randperm(E, generator=gen)[:2] for _ in range(n)]).reshape(-1)
            w = torch.rand(2 * n, 1, generator=gen)
            now = O.skip_now(True, state.skip, l, i, 2)
            # the test's own view of the policy (diep.py:61-68): enabled, an entry in the cache, an odd step
            assert now == (cache_rows[l] is not None and i % 2 != 0)
            cur.append((x, idx, w, "skip" if now else "full"))
            got = O.moe_infer_ep_async(state, x, layers[l], idx, w, 2, True, mask, now, l)
            if forced:
                ex, eidx, ew, kind = cur[l]
            elif pipeline:
                ex, eidx, ew, kind = hist[t - 1][l]
            else:
                ex, eidx, ew, kind = hist[max(t - 2, 0)][l]
            wt = (w if latest else ew).double().numpy().reshape(n, 2)
            x64 = ex.double().numpy()
            want = np.zeros((n, d))
            if kind == "full":
                rows_m = np.stack([_expert_row(layers[l], eidx[2 * tok + m], x64[tok]) for tok in range(n)])
                rows_r = np.stack([_expert_row(layers[l], eidx[2 * tok + r], x64[tok]) for tok in range(n)])
                cache_rows[l] = rows_m           # the put of a full emission: unweighted rows of the masked slots
            else:
                assert cache_rows[l] is not None, "a skip entry is emitted against an empty cache"
                rows_m = cache_rows[l]           # whatever expert the masked slot names now: the cached row stands
                rows_r = np.stack([_expert_row(layers[l], eidx[2 * tok + r], x64[tok]) for tok in range(n)])
                cache_rows[l] = None             # get empties the entry
            for tok in range(n):
                want[tok] = wt[tok, m] * rows_m[tok] + wt[tok, r] * rows_r[tok]
            assert got.shape == x.shape
            assert torch.allclose(got.double(), torch.from_numpy(want), atol=1e-4, rtol=1e-5), (t, l, kind)
        hist.append(cur)
        if forced:
            state.cancel_sync()
    kinds = [h[0][3] for h in hist]
    assert "skip" in kinds[1:] and "full" in kinds[1:], kinds


# --------------------------------------------------------------------------- #
# the block's caller: LayerNorm + modulate prologue, gated residual epilogue
# --------------------------------------------------------------------------- #
def test_norm_modulate_against_float64_definition():
    rng = np.random.default_rng(11)
    B, T, D = 3, 5, 48
    x = (rng.standard_normal((B, T, D)) * 3 + 2).astype(np.float32)
    shift = rng.standard_normal((B, D)).astype(np.float32)
    scale = rng.standard_normal((B, D)).astype(np.float32)
    x64 = x.astype(np.float64)
    mean = x64.mean(-1, keepdims=True)
    var = ((x64 - mean) ** 2).mean(-1, keepdims=True)          # biased
    want = (x64 - mean) / np.sqrt(var + 1e-6) * (1 + scale[:, None, :]) + shift[:, None, :]
    for single in (False, True):
        got = O.norm_modulate(torch.from_numpy(x), torch.from_numpy(shift), torch.from_numpy(scale),
                              single_rounding=single)
        assert np.allclose(got.double().numpy(), want, atol=2e-5, rtol=1e-5)
    # an unbiased variance or eps outside the root would miss by far more than the tolerance
    wrong = (x64 - mean) / np.sqrt(var * D / (D - 1) + 1e-6) * (1 + scale[:, None, :]) + shift[:, None, :]
    assert not np.allclose(wrong, want, atol=2e-5, rtol=1e-5)
    # constant rows normalise to zero: the output is the shift alone
    const = torch.full((B, T, D), 4.0)
    got = O.norm_modulate(const, torch.from_numpy(shift), torch.from_numpy(scale))
    assert torch.allclose(got, torch.from_numpy(shift)[:, None, :].expand(B, T, D), atol=1e-6)


def test_block_caller_identities():
    p = _small_block()
    g = torch.Generator().manual_seed(2)
    B, T, D = 2, 9, 64
    x = torch.randn(B, T, D, generator=g)
    shift, scale, gate = (torch.randn(B, D, generator=g) * 0.3 for _ in range(3))
    out, h, idx, wt, _ = O.dit_block_moe_half(p, x, shift, scale, gate)
    # definition, with the already pinned block on the already pinned prologue
    y, idx2, _, _ = O.sparse_moe_block_forward(p, h)
    assert torch.equal(idx, idx2)
    want = x.double() + gate.double()[:, None, :] * y.double()
    assert torch.allclose(out.double(), want, atol=1e-6)
    # gate = 0 leaves the stream untouched; scale = -1 feeds the layer the shift only
    out0, *_ = O.dit_block_moe_half(p, x, shift, scale, torch.zeros(B, D))
    assert torch.equal(out0, x)
    _, h1, *_ = O.dit_block_moe_half(p, x, shift, -torch.ones(B, D), gate)
    assert torch.allclose(h1, shift[:, None, :].expand(B, T, D), atol=1e-6)
    # fp32: one rounding or four, same result
    out_s, *_ = O.dit_block_moe_half(p, x, shift, scale, gate, single_rounding=True)
    assert torch.allclose(out_s, out, atol=1e-5)


def test_fp8_act_quantiser_non_finite_rows():
    """Build-defined: a row holding a NaN or an infinity quantises to zero bytes
    with a NaN scale (so every product of the row is NaN, as a 16-bit row would
    give); finite rows beside it are quantised as if it were not there."""
    g = torch.Generator().manual_seed(5)
    x = torch.randn(4, 64, generator=g)
    clean_q, clean_s = O.quantize_fp8_act(x)
    x[1, 3] = float("inf")
    x[2, 9] = float("nan")
    q, s = O.quantize_fp8_act(x)
    assert torch.isnan(s[1]) and torch.isnan(s[2]) and torch.isfinite(s[[0, 3]]).all()
    assert (q[1].float() == 0).all() and (q[2].float() == 0).all()
    assert torch.equal(q[[0, 3]].view(torch.uint8), clean_q[[0, 3]].view(torch.uint8))
    assert torch.equal(s[[0, 3]], clean_s[[0, 3]])
