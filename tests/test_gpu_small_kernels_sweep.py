"""Seeded sweeps over the latency-bound kernels in front of the expert GEMMs:
the router (both kernels: matrix pipe and dot products) and the dispatch (one
workgroup, two launches with the small-table and the general rank kernel,
three launches), at sizes around every switch between their code paths, with
ragged tails, skewed loads, empty experts, masks and illegal expert ids.

Router oracle: MoEGate.forward restated (reference models.py:179-196); dispatch
oracle: argsort(stable) + bincount + cumsum (models.py:365-367) with the slot
drop of a skip step (expertpara/ep_fwd.py:57-66).  Bars: indices, counts,
offsets and permutations bit-exact (router indices off the rows whose logits
tie within 1e-6), logits and weights to fp32 round-off."""
import pytest
import torch

from oracle import dice_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from dice_amd import lib
    lib.load()
    return torch.device("cuda:0")


def _gen(seed):
    return torch.Generator().manual_seed(seed)


# one case per line: tokens, hidden, experts, top-k, dtype, fp32 router matrix
ROUTER_CASES = [
    (1, 64, 2, 1, torch.bfloat16, False),        # a single token, two experts
    (31, 128, 8, 2, torch.bfloat16, False),      # less than one 32-token block
    (32, 128, 8, 2, torch.float16, False),
    (33, 256, 3, 2, torch.bfloat16, False),
    (1000, 384, 8, 2, torch.bfloat16, False),
    (4097, 1152, 8, 2, torch.bfloat16, False),
    (2500, 1152, 16, 4, torch.float16, False),
    (640, 2048, 16, 2, torch.bfloat16, False),   # eight waves per token block
    (640, 2304, 32, 6, torch.bfloat16, False),   # the longest rows the matrix-pipe router takes
    (640, 2368, 8, 2, torch.bfloat16, False),    # one chunk longer: the dot-product router
    (640, 1152, 33, 2, torch.bfloat16, False),   # one expert more than it takes
    (640, 1152, 8, 2, torch.bfloat16, True),     # fp32 router matrix for 16-bit activations
    (640, 1160, 8, 2, torch.bfloat16, False),    # hidden not a multiple of 64
    (777, 384, 8, 2, torch.float32, True),
    (129, 512, 64, 8, torch.float32, True),
]


@pytest.mark.parametrize("N,D,E,k,dtype,w32", ROUTER_CASES)
@pytest.mark.parametrize("skew", [False, True])
def test_router_sweep(dev, N, D, E, k, dtype, w32, skew):
    from dice_amd import ops
    g = _gen(N * 7 + D + E)
    x = torch.randn(N, D, generator=g).to(dtype)
    w = (torch.randn(E, D, generator=g) * 0.02)
    w = w if w32 else w.to(dtype)
    bias = None
    if skew:   # a Zipf-like load with (for E > 4) experts that nobody picks
        bias = torch.tensor([-(e ** 1.5) for e in range(E)], dtype=torch.float32)
    want_idx, want_w, want_logits = O.gate_forward(x, w, k, skew, bias)   # (skew also switches norm_topk_prob on)
    idx, wt, logits, idx64 = ops.gate_topk(x.to(dev), w.to(dev), k, skew, None if bias is None else bias.to(dev),
                                           want_logits=True, want_int64=True)
    idx, wt, logits, idx64 = idx.cpu(), wt.cpu(), logits.cpu(), idx64.cpu()
    assert torch.equal(idx64, idx.long())
    assert torch.allclose(logits, want_logits, atol=3e-5, rtol=1e-5)
    ties = O.gate_tie_rows(want_logits, k, tol=1e-6)
    assert torch.equal(idx.long()[~ties], want_idx[~ties]), "router indices differ off the tie rows"
    assert torch.allclose(wt[~ties], want_w[~ties], atol=1e-6, rtol=1e-5)
    assert ties.float().mean() < 0.02 or N < 64


def _check_dispatch(dev, idx, E, mask):
    from dice_amd import ops
    S = idx.numel()
    counts, offsets, perm, inv = ops.dispatch(idx.int().to(dev), E, None if mask is None else mask.to(dev))
    counts, offsets, perm, inv = counts.cpu().long(), offsets.cpu().long(), perm.cpu().long(), inv.cpu().long()
    legal = (idx >= 0) & (idx < E)
    kept_mask = legal if mask is None else legal & ~mask
    kept = kept_mask.nonzero().flatten()
    wc, wo, wp, _ = O.dispatch_tables(idx[kept], E)
    assert torch.equal(counts, wc)
    assert torch.equal(offsets, wo)
    n = kept.numel()
    assert torch.equal(perm[:n], kept[wp]), "perm differs from the stable argsort"
    assert (perm[n:] == -1).all()
    want_inv = torch.full((S,), -1, dtype=torch.long)
    want_inv[kept[wp]] = torch.arange(n)
    assert torch.equal(inv, want_inv)


# slots, experts: around 2048 slots (one workgroup / two launches), around 64 and 128
# spans of 256 slots and 8 / 16 experts (small-table rank kernels / the general one),
# and past spans^2 x experts = 4 M (three launches)
DISPATCH_CASES = [
    (2, 2), (64, 8), (65, 5), (2047, 8), (2048, 8), (2049, 8), (4000, 16),
    (16383, 8), (16384, 8), (16385, 8), (16384, 9), (16384, 16), (16385, 16), (16384, 17),
    (32768, 8), (32769, 8), (32768, 16), (40000, 7), (50000, 32), (131072, 8), (131072, 64),
    (185000, 8), (186000, 8), (262144, 16), (300001, 3),
]


@pytest.mark.parametrize("S,E", DISPATCH_CASES)
@pytest.mark.parametrize("load", ["uniform", "skewed", "one_expert"])
def test_dispatch_sweep(dev, S, E, load):
    g = _gen(S + 31 * E)
    if load == "uniform":
        idx = torch.randint(0, E, (S,), generator=g)
    elif load == "skewed":   # most slots on the first experts, the last ones empty
        idx = (torch.rand(S, generator=g) ** 3 * max(1, E - 2)).long()
    else:
        idx = torch.full((S,), E - 1, dtype=torch.long)
    _check_dispatch(dev, idx, E, None)
    mask = torch.rand(S, generator=g) < 0.5
    _check_dispatch(dev, idx, E, mask)
    if S >= 64:   # illegal expert ids are dropped like masked slots
        bad = idx.clone()
        bad[torch.randint(0, S, (S // 50 + 1,), generator=g)] = E + 3
        bad[torch.randint(0, S, (S // 50 + 1,), generator=g)] = -1
        _check_dispatch(dev, bad, E, mask)
