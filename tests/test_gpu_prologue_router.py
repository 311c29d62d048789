"""The caller's prologue with the router inside it (one launch for LayerNorm,
adaLN modulation and MoEGate.forward: reference models.py:75-76,497,519 and
179-196) against the same call with the two as separate launches, which the
other tests hold against the oracle.  Bar: bit-identical routing (indices and
weights) and output, since the fused kernel rounds the modulated rows the same
way and multiplies them with the router matrix in the same order; and the
routing against the oracle's on the oracle's own modulated rows, off the rows
whose logits tie."""
import pytest
import torch

from oracle import dice_oracle as O
from tests.helpers import block_from_params, router_own_launch, zipf_bias

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from dice_amd import lib
    lib.load()
    return torch.device("cuda:0")


def _run(blk, x, shift, scale, gate, eps=1e-6):
    from dice_amd.lib import CallerDesc, ptr
    B, T, D = x.shape
    c = CallerDesc()
    c.shift, c.scale, c.gate = ptr(shift), ptr(scale), ptr(gate)
    c.tokens_per_sample = T
    c.ln_eps = eps
    k = blk.num_experts_per_tok
    idx = torch.full((B * T, k), -7, dtype=torch.int32, device=x.device)
    wt = torch.full((B * T, k), -7.0, dtype=torch.float32, device=x.device)
    y = blk.run(x.view(-1, D), caller=c, topk_idx_out=idx, topk_weight_out=wt)
    torch.cuda.synchronize()
    return y.cpu(), idx.cpu(), wt.cpu()


# samples, tokens per sample, hidden, experts, top-k, dtype, router bias + normalised weights
CASES = [
    (32, 256, 1152, 8, 2, torch.bfloat16, False),   # the benchmark's block
    (3, 37, 384, 8, 2, torch.bfloat16, False),      # 111 tokens: a ragged last workgroup, workgroups that span samples
    (1, 1, 1152, 8, 2, torch.bfloat16, True),       # a single token
    (2, 50, 1536, 16, 4, torch.float16, True),      # the longest rows the kernel takes (eight router waves)
    (1, 33, 1024, 32, 6, torch.bfloat16, False),    # 32 experts
    (2, 40, 64, 3, 2, torch.float16, True),         # one chunk per 8 lanes, three experts
    (5, 64, 768, 8, 2, torch.float16, False),
    (2, 40, 2048, 8, 2, torch.bfloat16, False),     # longer rows: the call falls back to two launches
]


@pytest.mark.parametrize("B,T,D,E,k,dtype,skew", CASES)
def test_prologue_router_matches_separate_launches(dev, B, T, D, E, k, dtype, skew):
    g = torch.Generator().manual_seed(B * 1000 + T + D + E)
    bias = zipf_bias(E) if skew else None
    ratio = 1 if D >= 1024 else 2   # (narrow experts: this test is about the rows in front of them)
    p = O.make_block_params(D, E, k, ratio, ratio, seed=E + k, dtype=dtype, gate_bias=bias, norm_topk_prob=skew)
    blk = block_from_params(p, D, "swiglu", dtype, dev)
    x = (torch.randn(B, T, D, generator=g) * 2 + 0.5).to(dtype).to(dev)
    shift, scale, gate = ((torch.randn(B, D, generator=g) * 0.3).to(dtype).to(dev) for _ in range(3))
    y, idx, wt = _run(blk, x, shift, scale, gate)
    with router_own_launch():
        y2, idx2, wt2 = _run(blk, x, shift, scale, gate)
    assert torch.equal(idx, idx2), "routing differs from the router's own launch"
    assert torch.equal(wt, wt2)
    assert torch.equal(y, y2)
    assert torch.isfinite(y.float()).all()
    # the oracle's router on the oracle's modulated rows
    h = O.norm_modulate(x.cpu(), shift.cpu(), scale.cpu(), single_rounding=True).view(-1, D)
    want_idx, want_w, logits = O.gate_forward(h, p.gate_weight, k, skew, bias)
    # a one-ulp difference in a modulated element moves a logit by up to ~1e-3 in bf16
    ties = O.gate_tie_rows(logits, k, tol=2e-2)
    assert ties.float().mean() < 0.35 or B * T < 64
    assert torch.equal(idx.long()[~ties], want_idx[~ties])
    assert torch.allclose(wt[~ties], want_w[~ties], atol=2e-2)


def test_prologue_router_twice_and_smaller(dev):
    """Back-to-back calls on different token counts (the LDS tile and the partial
    logits of one workgroup must not leak into the next call's results)."""
    D, E, k = 1152, 8, 2
    p = O.make_block_params(D, E, k, 1, 1, seed=4, dtype=torch.bfloat16)
    blk = block_from_params(p, D, "swiglu", torch.bfloat16, dev)
    g = torch.Generator().manual_seed(77)
    for B, T in [(4, 256), (1, 45), (4, 256)]:
        x = torch.randn(B, T, D, generator=g).to(torch.bfloat16).to(dev)
        shift, scale, gate = ((torch.randn(B, D, generator=g) * 0.3).to(torch.bfloat16).to(dev) for _ in range(3))
        a = _run(blk, x, shift, scale, gate)
        with router_own_launch():
            b = _run(blk, x, shift, scale, gate)
        for u, v in zip(a, b):
            assert torch.equal(u, v)


def test_prologue_router_in_lagged_calls(dev):
    """Displaced mode through the fused caller: the prologue writes the modulated
    rows and the routing straight into the entry that outlives the call; four
    steps with the router inside the prologue equal four with it as its own
    launch, bit for bit."""
    from dice_amd import ParaMode, diep
    B, T, D = 2, 96, 256
    p = O.make_block_params(D, 8, 2, 2, 2, seed=3, dtype=torch.bfloat16, gate_std=0.1)
    pm = ParaMode(ep=True, ep_async=True, ep_async_mode="all")
    blk = block_from_params(p, D, "swiglu", torch.bfloat16, dev, para_mode=pm)

    def four_steps():
        diep.ep_cache_init(cache_capacity=1)
        diep.use_latest_expert_weights(True)
        outs = []
        try:
            for t in range(4):
                g = torch.Generator().manual_seed(20 + t)
                x = (torch.randn(B, T, D, generator=g) * 2 + 0.5).to(torch.bfloat16).to(dev)
                shift, scale, gate = ((torch.randn(B, D, generator=g) * 0.3).to(torch.bfloat16).to(dev)
                                      for _ in range(3))
                if t == 0:
                    diep.diep_force_sync()
                    diep.ep_cache_clear()
                outs.append(blk.forward_modulated(x, shift, scale, gate).cpu())
                if t == 0:
                    diep.diep_cancel_sync()
        finally:
            diep.ep_cache_init(cache_capacity=1)
            diep.use_latest_expert_weights(False)
            if diep.diep_forced_sync():
                diep.diep_cancel_sync()
        return outs

    a = four_steps()
    with router_own_launch():
        b = four_steps()
    for t, (u, v) in enumerate(zip(a, b)):
        assert torch.isfinite(u.float()).all()
        assert torch.equal(u, v), f"step {t}"
    assert not torch.equal(a[1], a[2])
