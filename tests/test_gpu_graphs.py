"""The layer recorded into a HIP graph: every replay must give what the same
call gives when launched directly, with the program's own eager work and
synchronisations between replays."""
import pytest
import torch

from oracle import dice_oracle as O
from tests.helpers import block_from_params

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from dice_amd import lib
    lib.load()
    return torch.device("cuda:0")


def _gen(seed):
    return torch.Generator().manual_seed(seed)


@pytest.mark.parametrize("D,N,dtype,variant", [
    (384, 1024, torch.float32, "swiglu"),      # DiT-S size, permutation-addressed fp32 kernels
    (384, 1024, torch.bfloat16, "gelu_tanh"),  # biased experts
    (1152, 2048, torch.bfloat16, "swiglu"),    # persistent kernels, tile tables built on the device
])
def test_graph_replays_match_eager(dev, D, N, dtype, variant):
    from dice_amd.graphs import GraphedBlock
    p = O.make_block_params(D, 8, 2, 4, 2, seed=21, dtype=dtype, variant=variant)
    blk = block_from_params(p, D, variant, dtype, dev)
    graphed = GraphedBlock(blk, N)
    for i in range(4):
        x = (torch.randn(N, D, generator=_gen(30 + i)) * (1 + i)).to(dtype).to(dev)
        want = blk.run(x)                 # eager launch between the replays
        torch.cuda.synchronize()
        got = graphed(x)
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay {i}"
        # routing changes from input to input: the graph must not have frozen it
        assert i == 0 or not torch.equal(got, first)
        first = got.clone() if i == 0 else first


def test_graph_survives_a_larger_eager_call(dev):
    """An eager call on more tokens makes the block size a new workspace; the
    recorded graph keeps the one it was recorded with."""
    from dice_amd.graphs import GraphedBlock
    D, N, dtype = 384, 512, torch.bfloat16
    p = O.make_block_params(D, 8, 2, 4, 2, seed=25, dtype=dtype)
    blk = block_from_params(p, D, "swiglu", dtype, dev)
    graphed = GraphedBlock(blk, N)
    x = torch.randn(N, D, generator=_gen(70)).to(dtype).to(dev)
    want = blk.run(x).clone()
    big = torch.randn(8 * N, D, generator=_gen(71)).to(dtype).to(dev)
    blk.run(big)                                    # new, larger workspace
    junk = [torch.full((1 << 20,), 7, dtype=torch.uint8, device=dev) for _ in range(8)]  # reuse freed memory, if any
    got = graphed(x)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    assert all(int(j.min()) == 7 and int(j.max()) == 7 for j in junk)


def test_graph_of_staleness_steps(dev):
    """A full step that fills the skip cache and a skip step that reads it, one
    graph each, alternating as the reference's schedule does."""
    from dice_amd.graphs import GraphedBlock
    from dice_amd.lib import MODE_PUT, MODE_SKIP
    D, N, dtype = 384, 512, torch.bfloat16
    p = O.make_block_params(D, 8, 2, 4, 2, seed=22, dtype=dtype)
    blk = block_from_params(p, D, "swiglu", dtype, dev)
    full, skip = GraphedBlock(blk, N, mode=MODE_PUT), GraphedBlock(blk, N, mode=MODE_SKIP)
    mask = torch.zeros(N * 2, dtype=torch.uint8, device=dev)
    mask[1::2] = 1
    full.skip_mask.copy_(mask)
    skip.skip_mask.copy_(mask)
    for i in range(3):
        x = torch.randn(N, D, generator=_gen(40 + i)).to(dtype).to(dev)
        cache = torch.empty_like(x)
        want_full = blk.run(x, MODE_PUT, mask, None, cache)
        got_full = full(x)
        torch.cuda.synchronize()
        assert torch.equal(got_full, want_full) and torch.equal(full.cache, cache)
        x2 = torch.randn(N, D, generator=_gen(50 + i)).to(dtype).to(dev)
        want_skip = blk.run(x2, MODE_SKIP, mask, cache, None)
        skip.cache.copy_(full.cache)
        got_skip = skip(x2)
        torch.cuda.synchronize()
        assert torch.equal(got_skip, want_skip), f"skip step {i}"


def test_graph_of_modulated_call(dev):
    from dice_amd.graphs import GraphedBlock
    B, T, D, dtype = 2, 256, 384, torch.bfloat16
    p = O.make_block_params(D, 8, 2, 4, 2, seed=23, dtype=dtype)
    blk = block_from_params(p, D, "swiglu", dtype, dev)
    graphed = GraphedBlock(blk, B * T, modulated=True, samples=B)
    for i in range(3):
        g = _gen(60 + i)
        x = torch.randn(B, T, D, generator=g).to(dtype).to(dev)
        shift, scale, gate = ((torch.randn(B, D, generator=g) * 0.3).to(dtype).to(dev) for _ in range(3))
        want = blk.forward_modulated(x, shift, scale, gate)
        got = graphed(x, shift, scale, gate)
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay {i}"


def test_graph_refuses_what_it_cannot_record(dev):
    from dice_amd import DiceError, ParaMode
    from dice_amd.graphs import GraphedBlock
    p = O.make_block_params(384, 8, 2, 4, 2, seed=24, dtype=torch.bfloat16)
    blk = block_from_params(p, 384, "swiglu", torch.bfloat16, dev)
    graphed = GraphedBlock(blk, 256)
    with pytest.raises(DiceError):
        graphed(torch.zeros(128, 384, dtype=torch.bfloat16, device=dev))
    lagged = block_from_params(p, 384, "swiglu", torch.bfloat16, dev, total_layers=4,
                               para_mode=ParaMode(ep=True, ep_async=True, num_sampling_steps=4))
    with pytest.raises(DiceError):
        GraphedBlock(lagged, 256)
