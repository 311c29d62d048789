"""GPU parity of the step-lagged layer calls (displaced / interweaved expert
parallelism on one GPU) against the oracle's restatement of the reference's
cache state machine, driven exactly as the reference's sampler drives it:
forced-sync first step with cleared caches, then lagged steps."""
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


def _reset(diep):
    diep.ep_cache_init(cache_capacity=1, noskip_step=1)
    diep.use_latest_expert_weights(False)
    if diep.diep_forced_sync():
        diep.diep_cancel_sync()


def _drive(dev, dtype, L, strategy, pipeline, latest, steps, D=256, E=8, N=384, noskip=1, skip_mode=None,
           tol=FP32_TOL, forced_at=(0,), drift=0.05):
    """Runs ``steps`` sampler steps over a stack of ``L`` blocks (layer l+1
    reads layer l's output plus a per-step drift, so every layer sees different
    inputs every step) on the GPU and in the oracle, comparing every output."""
    from dice_amd import ParaMode, diep
    params = [O.make_block_params(D, E, 2, 4, 2, seed=40 + l, gate_std=0.1, dtype=dtype) for l in range(L)]
    pm = ParaMode(ep=True, ep_async=True, ep_async_mode=strategy)
    blocks = [block_from_params(params[l], D, "swiglu", dtype, dev, layer_idx=l, total_layers=L, para_mode=pm)
              for l in range(L)]
    diep.ep_cache_init(cache_capacity=L, noskip_step=noskip, skip_mode=skip_mode, async_pipeline=pipeline,
                       selective_async_strategy=strategy)
    diep.use_latest_expert_weights(latest)
    diep.ep_set_rand_mask(None)
    state = O.DiepState(L, noskip_step=noskip, skip_mode=skip_mode, async_pipeline=pipeline,
                        selective_async_strategy=strategy, use_latest_expert_weights=latest)
    g = _gen(50)
    x0 = torch.randn(1, N, D, generator=g)
    try:
        for t in range(steps):
            i = steps - t                      # the reference counts steps down
            diep.ep_set_step(i)
            state.step = i
            forced = t in forced_at
            if forced:
                diep.diep_force_sync()
                diep.ep_cache_clear()
                state.force_sync()
                state.cache_clear()
            h_gpu = x0.to(dtype)
            for l in range(L):
                h_ref = h_gpu                  # both sides read the same layer input
                lagged = O.layer_is_async(strategy, l, L)
                want, _, _, logits = O.sparse_moe_block_forward(params[l], h_ref, state=state, async_op=lagged,
                                                                cache_key=l)
                y = blocks[l](h_ref.to(dev)).cpu()
                assert y.shape == want.shape
                err = rel_l2(y, want)
                assert err < tol, f"step {t} layer {l} forced={forced}: rel-L2 {err}"
                h_gpu = (want.float() * 0.5 + x0 * 0.5).to(dtype)
            if forced:
                diep.diep_cancel_sync()
                state.cancel_sync()
            x0 = (x0 if drift < 1.0 else 0.0) + drift * torch.randn(1, N, D, generator=g)
        assert diep.ep_cached_tensors_size() > 0
    finally:
        _reset(diep)


@pytest.mark.parametrize("latest", [False, True])
def test_displaced_fp32_follows_oracle(dev, latest):
    """Same layer, two steps of lag (one right after the forced-sync step):
    the recipe the reference's own test asserts (tests/test_ep.py:109-124)."""
    _drive(dev, torch.float32, L=2, strategy="all", pipeline=False, latest=latest, steps=5)


@pytest.mark.parametrize("strategy", ["all", "shallow", "deep", "interleaved"])
def test_interweaved_fp32_follows_oracle(dev, strategy):
    """Pipelined mode: a lagged layer runs the experts of the lagged layer
    before it and returns its own result of the previous step; a second
    forced-sync step in the middle (strided sync) refills the caches."""
    _drive(dev, torch.float32, L=4, strategy=strategy, pipeline=True, latest=True, steps=5, forced_at=(0, 3))


def test_displaced_bf16_persistent_path(dev):
    """bf16 at the width where the persistent 64-k kernels run (D=1152), so the
    lagged entry is read through its permutation by the fc1 kernel."""
    _drive(dev, torch.bfloat16, L=2, strategy="all", pipeline=False, latest=False, steps=4, D=1152, N=1024,
           tol=BF16_TOL)


def test_interweaved_bf16_persistent_path(dev):
    _drive(dev, torch.bfloat16, L=3, strategy="all", pipeline=True, latest=True, steps=4, D=1152, N=1024,
           tol=BF16_TOL)


@pytest.mark.parametrize("latest", [False, True])
@pytest.mark.parametrize("pipeline", [False, True])
@pytest.mark.parametrize("mode", ["high", "low"])
def test_lag_with_conditional_communication(dev, pipeline, mode, latest):
    """Step lag together with the skip cache at interval 2: whether a call
    blends with the cache or refills it follows the entry it returns, not the
    current step.  Every step draws a fresh input (no two steps alike, so the
    wrong entry, a stale cache row or the wrong routing weights cannot pass),
    with the cached and with the latest routing weights; the oracle's side of
    this sequence is pinned by the float64 closed form of
    tests/test_oracle.py::test_lag_with_skip_cache_closed_form."""
    _drive(dev, torch.float32, L=2, strategy="all", pipeline=pipeline, latest=latest, steps=9, noskip=2,
           skip_mode=mode, drift=1.0)


def test_lagged_equals_earlier_synchronous_result(dev):
    """Closed form at full C2 size, bf16, without the oracle: with the cached
    routing weights, the routed part of a displaced step's output is bit for
    bit the routed part the synchronous path produced two steps earlier (one
    step right after the forced-sync step); only the shared expert follows the
    current input."""
    from dice_amd import ParaMode, diep
    D, E, N = 1152, 8, 8192
    p = O.make_block_params(D, E, 2, 4, None, seed=9, dtype=torch.bfloat16)
    sync = block_from_params(p, D, "swiglu", torch.bfloat16, dev)
    pm = ParaMode(ep=True, ep_async=True, ep_async_mode="all")
    lag = block_from_params(p, D, "swiglu", torch.bfloat16, dev, para_mode=pm)
    g = _gen(11)
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
        # what stays cached: the newest entry (input copy + tables) and the one
        # before it, which has been through the experts (+ its rows)
        tables = (E + 1) * 4 + 3 * (2 * N) * 4
        assert diep.ep_cached_tensors_size() == 2 * (N * D * 2 + tables) + 2 * N * D * 2
    finally:
        _reset(diep)


def test_lagged_call_without_forced_sync_is_refused(dev):
    from dice_amd import ParaMode, diep
    D = 256
    p = O.make_block_params(D, 8, 2, 4, 2, seed=1)
    pm = ParaMode(ep=True, ep_async=True, ep_async_mode="all")
    blk = block_from_params(p, D, "swiglu", torch.float32, dev, para_mode=pm)
    diep.ep_cache_init(cache_capacity=1)
    try:
        with pytest.raises(AssertionError):
            blk(torch.randn(1, 64, D).to(dev))
    finally:
        _reset(diep)


def test_batch_change_between_lagged_steps_is_refused(dev):
    """A cached step only fits calls of its own shape: a different token count
    without a forced-sync step in between raises instead of reading the old
    tables out of range."""
    from dice_amd import DiceError, ParaMode, diep
    D = 256
    p = O.make_block_params(D, 8, 2, 4, 2, seed=1)
    pm = ParaMode(ep=True, ep_async=True, ep_async_mode="all")
    blk = block_from_params(p, D, "swiglu", torch.float32, dev, para_mode=pm)
    diep.ep_cache_init(cache_capacity=1)
    try:
        diep.diep_force_sync()
        blk(torch.randn(1, 64, D).to(dev))
        diep.diep_cancel_sync()
        with pytest.raises(DiceError, match="batch changes"):
            blk(torch.randn(1, 96, D).to(dev))
    finally:
        _reset(diep)


@pytest.mark.parametrize("async_op", [False, True])
@pytest.mark.parametrize("skip", [None, "high"])
def test_moe_infer_ep_function_follows_oracle(dev, async_op, skip):
    """The functional boundary of the reference (expertpara/ep_fwd.py:19) with
    the caller's own routing, driven like the reference's test of it
    (tests/test_ep.py:79-124): random expert ids (a token may name one expert
    twice) and random weights per iteration, forced-sync first iteration."""
    from dice_amd import ParaMode, diep
    from dice_amd.ep_fwd import moe_infer_ep
    D, E, N, k = 256, 8, 128, 2
    p = O.make_block_params(D, E, k, 4, None, seed=21)
    blk = block_from_params(p, D, "swiglu", torch.float32, dev, para_mode=ParaMode(ep=True))
    noskip = 2 if skip else 1
    diep.ep_cache_init(cache_capacity=1, noskip_step=noskip, skip_mode=skip)
    diep.use_latest_expert_weights(False)
    state = O.DiepState(1, noskip_step=noskip, skip_mode=skip)
    mask = O.skip_mask(N * k, skip) if skip else None
    g = _gen(60)
    try:
        for it in range(6):
            step = 6 - it
            diep.ep_set_step(step)
            state.step = step
            if it == 0:
                diep.diep_force_sync()
                diep.ep_cache_clear()
                state.force_sync()
                state.cache_clear()
            elif it == 1:
                diep.diep_cancel_sync()
                state.cancel_sync()
            x = torch.randn(N, D, generator=g)
            idx = torch.randint(0, E, (N * k,), generator=g)
            w = torch.rand(N * k, 1, generator=g)
            now = O.skip_now(True, state.skip, 0, step, noskip) if skip else None
            if skip:
                assert diep.ep_skip_now(0) == now
            want = O.moe_infer_ep_async(state, x, p.experts, idx, w, k, async_op, mask, now, 0)
            got = moe_infer_ep(x.to(dev), blk.experts, idx.to(dev), w.to(dev), k, async_op,
                               skip_mask=mask, skip_now=now, cache_key=0).cpu()
            assert rel_l2(got, want) < FP32_TOL, f"iteration {it}"
    finally:
        _reset(diep)


def test_displaced_f16_persistent_path(dev):
    """fp16, the dtype the reference serves its XL model in."""
    _drive(dev, torch.float16, L=2, strategy="all", pipeline=False, latest=True, steps=4, D=1152, N=1024,
           tol=4e-3)
