"""Benchmark of the MoE layer hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c1|c2|c3|c4|c5]
                    [--variant swiglu|gelu_tanh] [--activations bf16|fp8|fp8_blocks]

A step is one call of the whole layer (router -> dispatch -> grouped expert
MLP + shared expert -> combine) with inputs and weights resident in HBM.  The
default workload is the DiT-XL/2-MoE block (c2): 8192 tokens, hidden 1152, 8
experts, top-2, expert intermediate 4608, bf16 with fp32 accumulation.  The
other configurations (c1 DiT-S fp32, c3 16384 tokens with a Zipf-loaded router,
c4 the 50-step staleness loop, c5 DiT-G width with fp8 experts) run either as
the main workload (--config) or, in the default run, as short extra legs under
"configs".  Prints ONE JSON line.

    python bench.py [--config ...] --ab-hooks A B [--ab-call modulated] [--ab-lib other.so]

compares two settings "fc1,fc2" of the library's tuning hook (or two builds of the
library) on one block in an A B B A sequence of short segments instead, and
prints {"ab": ...}: us per call as mean and standard error, and whether the
outputs are bit-identical.
"""
import argparse
import json
import os
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"bf16": 2500.0, "fp8": 5000.0, "f32": 157.3}   # MI355X dense MFMA
PEAK_HBM_GBS = 8000.0

CONFIGS = {
    "c1": dict(name="DiT-S/2-MoE block (configs[0])", tokens=1024, samples=4, D=384, E=8, topk=2, ratio=4,
               dtype="f32"),
    "c2": dict(name="DiT-XL/2-MoE block (configs[1])", tokens=8192, samples=32, D=1152, E=8, topk=2, ratio=4,
               dtype="bf16"),
    "c3": dict(name="DiT-XL/2-MoE block at 512px, Zipf(1.2) router bias (configs[2])", tokens=16384, samples=16,
               D=1152, E=8, topk=2, ratio=4, dtype="bf16", zipf=1.2),
    "c4": dict(name="DiT-XL/2-MoE staleness loop, 50 steps (configs[3])", tokens=8192, samples=32, D=1152, E=8,
               topk=2, ratio=4, dtype="bf16", staleness=True),
    "c5": dict(name="DiT-G/2-MoE block, fp8 e4m3 routed experts (configs[4])", tokens=8192, samples=32, D=2048,
               E=16, topk=2, ratio=4, dtype="bf16", fp8=True),
}
TORCH_DTYPE = {"bf16": torch.bfloat16, "f32": torch.float32}
# rocprofv3 --pmc summaries of the dominant launch (bytes past the L2 per launch), keyed by (config, variant)
TRAFFIC_PROFILES = {("c2", "swiglu"): "profiles/layer_c2_bf16_hbm_traffic.txt",
                    ("c3", "swiglu"): "profiles/layer_c3_bf16_zipf_kernel_trace_and_mfma.txt",
                    ("c5", "swiglu"): "profiles/layer_c5_fp8_kernel_trace_and_counters.txt"}


def make_block(cfg, variant, dev, layer_idx=0, total_layers=1, para_mode=None, activations="bf16"):
    """Seeded synthetic weights: router N(0, 0.02), experts Xavier-uniform, zero biases."""
    from dice_amd import ParaMode, SparseMoeBlock
    D, E = cfg["D"], cfg["E"]
    # swiglu: the reference's shared expert (one SwiGLU MLP of width 2D, models.py:292-296);
    # gelu_tanh: two always-on experts of the routed shape = one MLP of width 2*4D.
    n_shared = 2 if variant == "swiglu" else 2 * cfg["ratio"]
    torch.manual_seed(layer_idx)
    with torch.device(dev):
        blk = SparseMoeBlock(D, cfg["ratio"], E, cfg["topk"], pretraining_tp=1, layer_idx=layer_idx,
                             total_layers=total_layers, para_mode=para_mode or ParaMode(), variant=variant,
                             n_shared_experts=n_shared)
    for m in blk.modules():
        if isinstance(m, torch.nn.Linear):
            torch.nn.init.xavier_uniform_(m.weight)
            if m.bias is not None:
                torch.nn.init.zeros_(m.bias)
    torch.nn.init.normal_(blk.gate.weight, std=0.02)
    blk = blk.to(device=dev, dtype=TORCH_DTYPE[cfg["dtype"]]).eval()
    if cfg.get("zipf"):
        pr = torch.tensor([(e + 1.0) ** -cfg["zipf"] for e in range(E)])
        blk.gate.bias = (pr / pr.sum()).log().float().to(dev)
    if cfg.get("fp8"):
        blk.quantize_fp8(activations=activations.startswith("fp8"), h_blocks=(activations == "fp8_blocks"))
    return blk


def make_input(cfg, dev, seed=0):
    x = torch.randn(cfg["tokens"], cfg["D"], generator=torch.Generator().manual_seed(seed))
    return x.to(TORCH_DTYPE[cfg["dtype"]]).to(dev)


def layer_flops(cfg, variant):
    n, D, k = cfg["tokens"], cfg["D"], cfg["topk"]
    slots, inter = n * k, cfg["ratio"] * D
    if variant == "swiglu":
        return {"fc1": 2.0 * slots * (2 * inter) * D, "fc2": 2.0 * slots * D * inter,
                "shared_fc1": 2.0 * n * (2 * 2 * D) * D, "shared_fc2": 2.0 * n * D * (2 * D)}
    return {"fc1": 2.0 * slots * inter * D, "fc2": 2.0 * slots * D * inter,
            "shared_fc1": 2.0 * n * (2 * inter) * D, "shared_fc2": 2.0 * n * D * (2 * inter)}


def _stage_names():
    from dice_amd.lib import load
    lib = load()
    n = lib.dice_profile_stage_count()
    return lib, n, [lib.dice_profile_stage_name(i).decode() for i in range(n)]


def time_layer(blk, x, steps, warmup):
    """Seconds per step over `steps` back-to-back layer calls, and the mean duration
    (ms) of the dominant launch (the routed fc1 expert GEMM) over the SAME calls: the
    library brackets that one launch with two HIP events per call on the stream it
    launches on (event rings of 64 calls, read without stopping the clock in between)."""
    import ctypes
    from dice_amd.lib import check
    lib, n, names = _stage_names()
    fc1 = names.index("moe.mlp.fc1")
    buf = (ctypes.c_float * n)()
    y = torch.empty_like(x)
    for _ in range(warmup):
        blk.run(x, y=y)
    check(lib.dice_profile_enable(2))
    fc1_ms, done = 0.0, 0
    try:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while done < steps:
            chunk = min(64, steps - done)
            for _ in range(chunk):
                blk.run(x, y=y)
            if done + chunk < steps:
                check(lib.dice_profile_read(buf, n))   # waits for this chunk's last fc1 only
                fc1_ms += buf[fc1] * chunk
            done += chunk
        torch.cuda.synchronize()
        sec = (time.perf_counter() - t0) / steps
        last = steps - (steps - 1) // 64 * 64
        check(lib.dice_profile_read(buf, n))
        fc1_ms += buf[fc1] * last
    finally:
        check(lib.dice_profile_enable(0))
    return sec, fc1_ms / steps


def time_after_idle(blk, x, calls=64, idle_s=2.0):
    """Duration (ms) of each of the first `calls` layer calls after `idle_s` seconds without GPU work, from
    one event per call on torch's current stream.  A run of 20 timed steps behind 5 warm-ups falls into the
    transient this shows (the board's power management answering a step from idle to full load), a longer run
    averages over it."""
    y = torch.empty_like(x)
    torch.cuda.synchronize()
    time.sleep(idle_s)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(calls + 1)]
    ev[0].record()
    for i in range(calls):
        blk.run(x, y=y)
        ev[i + 1].record()
    torch.cuda.synchronize()
    return [round(ev[i].elapsed_time(ev[i + 1]), 4) for i in range(calls)]


def time_batch_sizes(cfg, variant, dev, sizes=(256, 1024, 1536, 2048, 4096), calls=200):
    """ms per layer call of the same block at other token counts (sampling batches of 1 to 16 images):
    `calls` back-to-back calls after 20 warm-ups each."""
    out = {}
    for n in sizes:
        c = dict(cfg)
        c["tokens"], c["samples"] = n, max(1, n // 256)
        blk = make_block(c, variant, dev)
        x = make_input(c, dev)
        y = torch.empty_like(x)
        for _ in range(20):
            blk.run(x, y=y)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(calls):
            blk.run(x, y=y)
        torch.cuda.synchronize()
        out[str(n)] = round((time.perf_counter() - t0) / calls * 1e3, 5)
        del blk, x, y
    return out


def time_stages(blk, x, steps):
    """Mean duration of every launch of the layer in ms, from the library's own
    stage timers: HIP events recorded between the launches of dice_moe_forward
    on the stream it launches on (torch's current stream)."""
    import ctypes
    from dice_amd.lib import check
    lib, n, names = _stage_names()
    check(lib.dice_profile_enable(1))
    buf = (ctypes.c_float * n)()
    acc = [0.0] * n
    y = torch.empty_like(x)
    # Back-to-back calls, read once per chunk of at most 64 (the library's event ring):
    # the same sustained regime as the timed region, not cooled by a host wait per call.
    done = 0
    try:
        for _ in range(2):
            blk.run(x, y=y)
        check(lib.dice_profile_read(buf, n))
        while done < steps:
            chunk = min(64, steps - done)
            for _ in range(chunk):
                blk.run(x, y=y)
            check(lib.dice_profile_read(buf, n))
            for i in range(n):
                acc[i] += buf[i] * chunk
            done += chunk
    finally:
        check(lib.dice_profile_enable(0))
    return {names[i]: acc[i] / steps for i in range(n)}


def hbm_stage_bytes(cfg, es):
    """Algorithmic bytes of the bandwidth-bound launches of a plain step."""
    n, D, k = cfg["tokens"], cfg["D"], cfg["topk"]
    slots = n * k
    return {"moe.gate": n * D * es + slots * 8,
            "moe.dispatch": slots * 12,
            "moe.combine": (slots * D + 2 * n * D) * es + slots * 8}


def staleness_schedule(sample_steps):
    """The reference sampler's countdown (diffusion/rectified_flow.py:83-105): yields (step, clear)."""
    from dice_amd import diep
    for i in range(sample_steps, 0, -1):
        yield i, diep.ep_forced_sync(i, sample_steps)


def time_staleness(cfg, variant, dev, x, sample_steps=50, modes=("high", "low", "rand")):
    """Configuration 4: the conditional-communication loop of the reference sampler on this
    layer: 50 steps counted down, the first a full step, then skip steps (one routed slot per
    token recomputed, the other read from the per-layer cache in the combine) alternating with
    full steps that refill the cache; x drifts by 0.05 N(0,1) per step.  No host synchronisation
    inside the loop: every layer call is bracketed by two events on the stream it runs on, the
    whole loop by the host clock.  A second pass reads the library's stage timers after every
    step and gives the sum of a step's kernels per step kind; a third runs the config-literal
    form (a resident foreign N(0,1) cache, every step a skip step)."""
    import ctypes
    from dice_amd import ParaMode, diep, lib as L
    from dice_amd.lib import check
    blk = make_block(cfg, variant, dev, 0, 1, ParaMode(ep=True))
    n_tok, D = cfg["tokens"], cfg["D"]
    xv = x.view(1, n_tok, D)
    g = torch.Generator(device=dev).manual_seed(4)
    noise = [0.05 * torch.randn(xv.shape, generator=g, device=dev, dtype=torch.float32) for _ in range(4)]
    lib, n, names = _stage_names()
    buf = (ctypes.c_float * n)()
    out = {}
    try:
        for mode in modes:
            diep.ep_cache_init(cache_capacity=1, noskip_step=2, skip_mode=mode)
            diep.ep_set_rand_mask(None)
            ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
                  for _ in range(sample_steps)]
            kinds = []
            wall = 0.0
            for rep in range(2):            # first repetition warms up
                xt = xv.clone()
                kinds = []
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for j, (i, clear) in enumerate(staleness_schedule(sample_steps)):
                    diep.ep_set_step(i)
                    if clear:
                        diep.ep_cache_clear()
                    kinds.append("skip" if diep.ep_skip_now(0) else "full")
                    ev[j][0].record()
                    blk(xt)
                    ev[j][1].record()
                    xt = (xt.float() + noise[i % 4]).to(xt.dtype)
                torch.cuda.synchronize()
                wall = time.perf_counter() - t0
            per = {"full": [], "skip": []}
            for j, kd in enumerate(kinds):
                per[kd].append(ev[j][0].elapsed_time(ev[j][1]))
            res = {"ms_per_step": sum(sum(v) for v in per.values()) / sample_steps,
                   "loop_wall_ms_per_step_incl_drift_update": wall / sample_steps * 1e3,
                   "full_put_step_ms": statistics.mean(per["full"]), "skip_step_ms": statistics.mean(per["skip"]),
                   "full_steps": len(per["full"]), "skip_steps": len(per["skip"])}
            # second pass: the kernels of each step kind, from the stage timers
            check(lib.dice_profile_enable(1))
            try:
                ksum = {"full": [], "skip": []}
                stages = {"full": [0.0] * n, "skip": [0.0] * n}
                xt = xv.clone()
                for i, clear in staleness_schedule(sample_steps):
                    diep.ep_set_step(i)
                    if clear:
                        diep.ep_cache_clear()
                    kd = "skip" if diep.ep_skip_now(0) else "full"
                    blk(xt)
                    check(lib.dice_profile_read(buf, n))
                    ksum[kd].append(sum(buf))
                    for q in range(n):
                        stages[kd][q] += buf[q]
                    xt = (xt.float() + noise[i % 4]).to(xt.dtype)
            finally:
                check(lib.dice_profile_enable(0))
            res["full_put_step_kernels_ms"] = statistics.mean(ksum["full"])
            res["skip_step_kernels_ms"] = statistics.mean(ksum["skip"])
            res["skip_step_stage_ms"] = {names[q]: stages["skip"][q] / len(ksum["skip"]) for q in range(n)}
            es = x.element_size()
            # combine of a skip step: one fresh slot row, the cached row and the shared row in, one row out
            comb = (n_tok * D * 4) * es + n_tok * cfg["topk"] * 9
            res["skip_combine_gbs"] = comb / (res["skip_step_stage_ms"]["moe.combine"] * 1e-3) / 1e9
            out[mode] = res
        # config-literal form: a foreign cache stays resident, every step is a skip step against it
        diep.ep_cache_init(cache_capacity=1, noskip_step=2, skip_mode="high")
        mask = diep.ep_skip_mask_on(n_tok * cfg["topk"], dev)
        cache = torch.randn(n_tok, D, generator=g, device=dev, dtype=torch.float32).to(x.dtype)
        y = torch.empty_like(x)
        xt = x.clone()
        for rep in range(2):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for i in range(sample_steps):
                blk.run(xt, L.MODE_SKIP, mask, cache, None, y=y)
                xt = (xt.float() + noise[i % 4][0]).to(xt.dtype)
            torch.cuda.synchronize()
            wall = time.perf_counter() - t0
        out["every_step_skip_resident_cache_high"] = {"loop_wall_ms_per_step_incl_drift_update": wall / sample_steps * 1e3}
    finally:
        diep.ep_cache_init(cache_capacity=1, noskip_step=1)
    return out


def time_sustained_cold(cfg, variant, dev, n_blocks=8, seconds=1.0):
    """What the reference's sampler makes of the layer: a stack of blocks with distinct weights,
    each with its own input, walked in order again and again (models.py:653-688 walks `depth`
    blocks per step).  `n_blocks` blocks of this configuration (8 x 271 MB of weights at C2:
    beyond the 256 MB memory-side cache, so every call streams its weights from HBM) are
    called round-robin for at least `seconds`, with no host synchronisation inside a group
    of 64 calls; the dominant launch is bracketed by the library's two HIP events per call
    over the SAME run.  Returns whole-run throughput and that launch's mean duration."""
    import ctypes
    from dice_amd.lib import check
    lib, n, names = _stage_names()
    fc1 = names.index("moe.mlp.fc1")
    buf = (ctypes.c_float * n)()
    blocks = [make_block(cfg, variant, dev, layer_idx=l, total_layers=n_blocks) for l in range(n_blocks)]
    xs = [make_input(cfg, dev, seed=100 + l) for l in range(n_blocks)]
    ys = [torch.empty_like(x) for x in xs]
    weight_bytes = 0
    for b in blocks:
        b.run(xs[0], y=ys[0])        # packs the weights, sizes the workspace
        pk = b._packed
        weight_bytes += sum(t.numel() * t.element_size() for t in (pk.w1, pk.w2, pk.sw1, pk.sw2) if t is not None)
    for l, b in enumerate(blocks):   # one untimed walk
        b.run(xs[l], y=ys[l])
    check(lib.dice_profile_enable(2))
    calls, fc1_ms = 0, 0.0
    rounds_per_group = max(1, 64 // n_blocks)
    try:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while True:
            for _ in range(rounds_per_group):
                for l, b in enumerate(blocks):
                    b.run(xs[l], y=ys[l])
            group = rounds_per_group * n_blocks
            check(lib.dice_profile_read(buf, n))   # waits for this group's last fc1 launch only
            fc1_ms += buf[fc1] * group
            calls += group
            if time.perf_counter() - t0 >= seconds:
                break
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
    finally:
        check(lib.dice_profile_enable(0))
    del blocks, xs, ys
    torch.cuda.empty_cache()
    return {"blocks": n_blocks, "distinct_weight_bytes": weight_bytes, "calls": calls, "seconds": wall,
            "ms_per_step": wall / calls * 1e3, "tokens_per_s": cfg["tokens"] * calls / wall,
            "fc1_ms_per_launch": fc1_ms / calls}


def time_staleness_layers(cfg, variant, dev, n_layers=8, sample_steps=50, mode="high"):
    """The staleness loop as the reference runs it: `n_layers` blocks with distinct weights and
    one skip-cache entry per layer (cache_capacity = depth, sample_ddp.py:182-192), every
    sampler step walking all of them; layer l has its own drifting input.  Milliseconds per
    layer call over the whole loop (host clock, no synchronisation inside) and per step kind
    (two events per layer call)."""
    from dice_amd import ParaMode, diep
    n_tok, D = cfg["tokens"], cfg["D"]
    blocks = [make_block(cfg, variant, dev, l, n_layers, ParaMode(ep=True)) for l in range(n_layers)]
    g = torch.Generator(device=dev).manual_seed(5)
    noise = [0.05 * torch.randn((1, n_tok, D), generator=g, device=dev, dtype=torch.float32) for _ in range(4)]
    x0 = [make_input(cfg, dev, seed=200 + l).view(1, n_tok, D) for l in range(n_layers)]
    try:
        diep.ep_cache_init(cache_capacity=n_layers, noskip_step=2, skip_mode=mode)
        diep.ep_set_rand_mask(None)
        ev = [[(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n_layers)]
              for _ in range(sample_steps)]
        kinds, wall = [], 0.0
        for rep in range(2):            # first repetition warms up
            xt = [x.clone() for x in x0]
            kinds = []
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for j, (i, clear) in enumerate(staleness_schedule(sample_steps)):
                diep.ep_set_step(i)
                if clear:
                    diep.ep_cache_clear()
                kinds.append("skip" if diep.ep_skip_now(0) else "full")
                for l, b in enumerate(blocks):
                    ev[j][l][0].record()
                    b(xt[l])
                    ev[j][l][1].record()
                    xt[l] = (xt[l].float() + noise[(i + l) % 4]).to(xt[l].dtype)
            torch.cuda.synchronize()
            wall = time.perf_counter() - t0
        per = {"full": [], "skip": []}
        for j, kd in enumerate(kinds):
            per[kd].extend(ev[j][l][0].elapsed_time(ev[j][l][1]) for l in range(n_layers))
        cached = diep.ep_cached_tensors_size()
    finally:
        diep.ep_cache_init(cache_capacity=1, noskip_step=1)
    del blocks
    torch.cuda.empty_cache()
    calls = sample_steps * n_layers
    return {"layers": n_layers, "skip_mode": mode, "ms_per_layer_call": sum(sum(v) for v in per.values()) / calls,
            "loop_wall_ms_per_layer_call_incl_drift_update": wall / calls * 1e3,
            "full_put_step_ms_per_layer_call": statistics.mean(per["full"]),
            "skip_step_ms_per_layer_call": statistics.mean(per["skip"]),
            "full_steps": kinds.count("full"), "skip_steps": kinds.count("skip"), "cached_bytes_at_end": cached}


def time_lagged(cfg, variant, dev, x, steps, warmup, pipeline):
    """ms per layer call of the step-lagged modes on the same block shape: two
    layers, a forced-sync first step, then `steps` lagged steps (displaced: each
    layer two steps behind itself; interweaved: each layer runs the other one's
    experts and is one step behind).  Includes the per-call copy of the layer
    input into the cached entry."""
    from dice_amd import ParaMode, diep
    pm = ParaMode(ep=True, ep_async=True, ep_async_mode="all")
    blks = [make_block(cfg, variant, dev, l, 2, pm) for l in range(2)]
    diep.ep_cache_init(cache_capacity=2, async_pipeline=pipeline, selective_async_strategy="all")
    diep.use_latest_expert_weights(True)
    xv = x.view(1, cfg["tokens"], cfg["D"])
    try:
        diep.diep_force_sync()
        diep.ep_cache_clear()
        for b in blks:
            b(xv)
        diep.diep_cancel_sync()
        for _ in range(warmup):
            for b in blks:
                b(xv)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            for b in blks:
                b(xv)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / (steps * len(blks)) * 1e3
    finally:
        diep.ep_cache_init(cache_capacity=1)
        diep.use_latest_expert_weights(False)


def time_caller(cfg, blk, x, steps, warmup, hook=(0, 0)):
    """The MoE line of the reference's DiTBlock.forward, x + gate * moe(modulate(norm2(x))):
    ms per call with the prologue / epilogue inside the library, with them as torch eager ops
    around the plain layer call (what the reference's DiTBlock does), and the prologue kernel
    alone with its share of the 8 TB/s HBM peak."""
    import torch.nn.functional as F
    from dice_amd import ops
    B, D = cfg["samples"], cfg["D"]
    g = torch.Generator().manual_seed(1)
    xs = x.view(B, cfg["tokens"] // B, D)
    shift, scale, gate = ((torch.randn(B, D, generator=g) * 0.3).to(x.dtype).to(x.device) for _ in range(3))
    out = torch.empty_like(xs)

    def fused():
        blk.forward_modulated(xs, shift, scale, gate, out=out)

    def eager():
        h = F.layer_norm(xs, (D,), None, None, 1e-6) * (1 + scale.unsqueeze(1)) + shift.unsqueeze(1)
        return xs + gate.unsqueeze(1) * blk(h)

    def prologue():
        ops.ln_modulate(xs, shift, scale)

    from dice_amd import lib
    # "fused": the library's call (prologue and router in one launch); "fused_router_own_launch":
    # the same call with the router as a launch of its own (tuning hook).  The board's clocks
    # drift with the load of the last few milliseconds (a leg that follows a light one ran 1-2 %
    # slower than the same leg elsewhere), so the three layer-call legs take turns in short
    # rounds, one round per order of the three, and the prologue-only leg runs after them.
    import itertools
    legs = {"fused": fused, "fused_router_own_launch": fused, "eager_caller": eager}
    orders = list(itertools.permutations(legs))
    per_round = max(1, steps // len(orders))
    total = {name: 0.0 for name in legs}
    for r, order in enumerate(orders):
        for name in order:
            if name == "fused_router_own_launch":
                lib.load().dice_set_gemm_config(50, hook[1])
            try:
                for _ in range(warmup if r == 0 else 2):
                    legs[name]()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(per_round):
                    legs[name]()
                torch.cuda.synchronize()
                total[name] += time.perf_counter() - t0
            finally:
                if name == "fused_router_own_launch":
                    lib.load().dice_set_gemm_config(*hook)
    res = {name: total[name] / (len(orders) * per_round) * 1e3 for name in legs}
    for _ in range(warmup):
        prologue()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(20 * steps):   # (a 10 us kernel: many calls per wait)
        prologue()
    torch.cuda.synchronize()
    res["ln_modulate_kernel"] = (time.perf_counter() - t0) / (20 * steps) * 1e3
    res["ln_modulate_frac_of_hbm_peak"] = (2 * cfg["tokens"] * D * x.element_size()
                                           / (res["ln_modulate_kernel"] * 1e-3) / 1e9 / PEAK_HBM_GBS)
    return res


def cpu_threads():
    """Threads for the CPU baseline: the host's cores, capped by the thread count the
    environment grants (OMP_NUM_THREADS: a GPU box shares its cores between its GPUs)."""
    have = os.cpu_count() or 1
    env = os.environ.get("OMP_NUM_THREADS", "")
    return min(have, int(env)) if env.isdigit() and int(env) > 0 else have


def cpu_baseline(cfg, variant, budget_s=10.0, dtypes=None):
    """The oracle (a torch restatement of the reference block) timed on the host cores on a
    bounded token sample of the same workload, in the workload's dtype and, for 16-bit
    workloads, in fp32 as well (CPU bf16 GEMM speed depends on the ISA).  The headline
    `value` is the faster leg."""
    from oracle import dice_oracle as O
    cores = cpu_threads()
    torch.set_num_threads(cores)
    D, E, k, n_tok = cfg["D"], cfg["E"], cfg["topk"], cfg["tokens"]
    n_shared = 2 if variant == "swiglu" else 2 * cfg["ratio"]
    legs = {}
    for name in dtypes or ([cfg["dtype"], "f32"] if cfg["dtype"] != "f32" else ["f32"]):
        dt = TORCH_DTYPE[name]
        bias = None
        if cfg.get("zipf"):
            pr = torch.tensor([(e + 1.0) ** -cfg["zipf"] for e in range(E)])
            bias = (pr / pr.sum()).log()
        p = O.make_block_params(D, E, k, cfg["ratio"], n_shared, seed=0, dtype=dt, variant=variant, gate_bias=bias)
        g = torch.Generator().manual_seed(1)
        probe = torch.randn(1, 256, D, generator=g).to(dt)
        O.sparse_moe_block_forward(p, probe)
        t0 = time.perf_counter()
        O.sparse_moe_block_forward(p, probe)
        per_tok = (time.perf_counter() - t0) / 256
        sample = int(min(n_tok, max(256, (budget_s / 4) / max(per_tok, 1e-9))))
        sample = max(256, sample // 256 * 256)
        xs = torch.randn(1, sample, D, generator=g).to(dt)
        t0 = time.perf_counter()
        O.sparse_moe_block_forward(p, xs)
        first = time.perf_counter() - t0
        reps = int(max(3, min(200, (budget_s / 2) / max(first, 1e-6))))
        times = []
        for _ in range(reps):
            t0 = time.perf_counter()
            O.sparse_moe_block_forward(p, xs)
            times.append(time.perf_counter() - t0)
        t = statistics.median(times)
        legs[name] = {"tokens_per_s": sample / t, "sample_tokens": sample, "calls": reps, "s_per_call": t,
                      "cpu_work_s": sum(times) + first}
    best = max(legs, key=lambda q: legs[q]["tokens_per_s"])
    return {"value": legs[best]["tokens_per_s"], "unit": "tokens/s", "cores": cores, "kind": "port",
            "dtype": best, "legs": legs, "host_cpu_count": os.cpu_count(),
            "parallel_info": " ".join(torch.__config__.parallel_info().split()),
            "sample": f"{legs[best]['sample_tokens']} of {n_tok} tokens per call (tokens are independent), torch "
                      f"oracle of the reference block in {best}, median of {legs[best]['calls']} calls after 2 "
                      f"warm-ups, {legs[best]['s_per_call']:.3f} s each; {sum(l['cpu_work_s'] for l in legs.values()):.1f}"
                      f" s of CPU work over {len(legs)} dtype legs on {cores} threads"}


def time_vendor_gemm(cfg, blk, x, dev):
    """What the vendor's GEMM (torch.matmul -> hipBLASLt) reaches on this board, which is power-limited for
    bf16 matrix work so that throughput depends on the operand values: the routed fc1 as ONE plain GEMM
    ([N*k, D] x [2I, D]^T, no activation, no gather, no shared expert) on this run's activations and the first
    expert's weights, and an 8192^3 GEMM on N(0,1) operands.  A reference for `roofline.achieved`, not a part
    of the layer."""
    def run(a, b, reps=20):
        c = torch.empty(a.shape[0], b.shape[0], dtype=a.dtype, device=dev)
        for _ in range(3):
            torch.matmul(a, b.t(), out=c)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            torch.matmul(a, b.t(), out=c)
        torch.cuda.synchronize()
        return 2.0 * a.shape[0] * b.shape[0] * a.shape[1] / ((time.perf_counter() - t0) / reps) / 1e12
    a = x.repeat(cfg["topk"], 1)
    w1 = blk._packed.w1[0]
    if w1.dtype != a.dtype:
        return None
    big = torch.randn(8192, 8192, device=dev).to(x.dtype)
    return {"routed_fc1_shape_%dx%dx%d" % (a.shape[0], w1.shape[0], a.shape[1]): run(a, w1),
            "8192x8192x8192_randn": run(big, big)}


def workload_text(cfg, variant, activations):
    D, inter = cfg["D"], cfg["ratio"] * cfg["D"]
    shared = f"{D}->{2 * D}->{D} (reference)" if variant == "swiglu" else f"2 x ({D}->{inter}->{D})"
    if cfg.get("fp8"):
        prec = ("routed experts e4m3 weights (per-output-channel scales), "
                + ("activations quantised per token to e4m3 in front of each GEMM, fp8 MFMA" if activations == "fp8"
                   else "x quantised per token to e4m3, h per token and 32 columns inside fc1's epilogue (power-of-two "
                        "scales, scaled fp8 MFMA in fc2)" if activations == "fp8_blocks"
                   else "bf16 activations (weights widened, bf16 MFMA)")
                + ", shared expert bf16")
    else:
        prec = f"{cfg['dtype']} in/out, fp32 accumulate"
    return (f"{cfg['name']}: {cfg['tokens']} tokens x {D}, {cfg['E']} experts top-{cfg['topk']}, expert "
            f"{D}->{inter}->{D} {variant}, shared expert {shared}, {prec}")


def measure(cfg_name, variant, activations, dev, steps, warmup, stages=True):
    """One configuration: throughput of the layer call and the roofline of its dominant launch."""
    cfg = CONFIGS[cfg_name]
    blk = make_block(cfg, variant, dev, activations=activations)
    x = make_input(cfg, dev)
    sec, fc1_ms = time_layer(blk, x, steps, warmup)
    flops = layer_flops(cfg, variant)
    total_flops = sum(flops.values())
    a8 = bool(cfg.get("fp8")) and activations.startswith("fp8")
    pipe = "fp8" if a8 else cfg["dtype"]
    res = {"tokens_per_s": cfg["tokens"] / sec, "ms_per_step": sec * 1e3, "workload": workload_text(cfg, variant, activations),
           "layer_tflops": total_flops / sec / 1e12}
    # Dominant kernel: the routed fc1 launch (activation fused; with 16-bit weights the shared
    # expert's fc1 rides in the same launch), timed inside the timed region above.
    joint = not cfg.get("fp8") and cfg["dtype"] != "f32"
    dom_flops = flops["fc1"] + (flops["shared_fc1"] if joint else 0.0)
    swiglu = variant == "swiglu"
    if fc1_ms > 0:
        ach = dom_flops / (fc1_ms * 1e-3) / 1e12
        kern = ("gemm_persist_kernel_f8" if a8 else "gemm_persist_kernel4") if cfg["dtype"] != "f32" else "grouped_gemm_f32_kernel"
        res["roofline"] = {"bound": "mfma",
                           "kernel": "%s<fc1 %s> (routed%s fc1, activation fused)"
                                     % (kern, "SwiGLU" if swiglu else "GELU-tanh, biased", " + shared expert" if joint else ""),
                           "achieved": ach, "peak": PEAK_TFLOPS[pipe], "unit": "TFLOP/s", "frac": ach / PEAK_TFLOPS[pipe],
                           "traffic": None, "flop_per_launch": dom_flops, "ms_per_launch": fc1_ms}
        prof = TRAFFIC_PROFILES.get((cfg_name, variant))
        if prof and os.path.exists(os.path.join(ROOT, prof)):
            # (not measured in this run: the figure of the committed rocprofv3 --pmc summary of this command)
            for line in open(os.path.join(ROOT, prof)):
                if line.startswith("traffic_bytes_per_launch:"):
                    res["roofline"]["traffic"] = float(line.split(":")[1])
                    res["roofline"]["traffic_source"] = prof
    if stages:
        st = time_stages(blk, x, max(5, steps))
        res["stage_ms"] = st
        gemm_ms = sum(st[s] for s in ("moe.mlp.fc1", "moe.mlp.shared_fc1", "moe.mlp.fc2", "moe.mlp.shared_fc2"))
        if gemm_ms > 0:
            res["mfma_util_pct_of_peak"] = 100.0 * total_flops / (gemm_ms * 1e-3) / 1e12 / PEAK_TFLOPS[cfg["dtype"]]
        if a8:
            # the two fp8 launches against the fp8 peak, and what the quantisers in front of them move
            res["fp8_launch_frac_of_fp8_peak"] = {
                "fc1": flops["fc1"] / (st["moe.mlp.fc1"] * 1e-3) / 1e12 / PEAK_TFLOPS["fp8"],
                "fc2": flops["fc2"] / (st["moe.mlp.fc2"] * 1e-3) / 1e12 / PEAK_TFLOPS["fp8"]}
            slots, D, inter = cfg["tokens"] * cfg["topk"], cfg["D"], cfg["ratio"] * cfg["D"]
            res["quantiser_gbs"] = {"x": slots * D * 3 / (st["moe.gather"] * 1e-3) / 1e9,
                                    "h": slots * inter * 3 / (st["moe.quant_h"] * 1e-3) / 1e9
                                    if activations == "fp8" else None}
        hbm = hbm_stage_bytes(cfg, x.element_size())
        res["hbm_stage_gbs"] = {s: hbm[s] / (st[s] * 1e-3) / 1e9 for s in hbm if st[s] > 0}
        res["hbm_stage_frac_of_peak"] = {s: v / PEAK_HBM_GBS for s, v in res["hbm_stage_gbs"].items()}
    return cfg, blk, x, res


def ab_hooks(cfg_name, variant, activations, dev, hook_a, hook_b, lib_b=None, call="layer", tokens=None,
             groups=12, seg=20):
    """Two settings of the tuning hook (or two builds of the library: `lib_b` names the other
    .so) on the same block in one process, in an A B B A sequence of `groups` x 4 segments of
    `seg` back-to-back calls each; us per call as mean and standard error over the segments.
    The board's clocks drift with the load of the last milliseconds, so that timing one
    setting after the other compares their places in the run rather than the settings."""
    import ctypes
    import statistics
    from dice_amd import lib
    from dice_amd.lib import CallerDesc, ptr, stream_ptr
    cfg = dict(CONFIGS[cfg_name])
    if tokens:                                        # another batch size of the same block
        cfg["tokens"] = tokens
        cfg["samples"] = max(1, tokens // 256)
    blk = make_block(cfg, variant, dev, activations=activations)
    x = make_input(cfg, dev)
    y = torch.empty_like(x)
    blk.run(x, y=y)                                   # packs the weights, sizes the workspace
    desc = blk._ensure(x)
    ws = blk._workspace(desc, x.shape[0], x.device)
    libs = [lib.load(), lib.load()]
    if lib_b:
        other = ctypes.CDLL(os.path.abspath(lib_b))
        for name in ("dice_moe_forward", "dice_moe_forward_modulated", "dice_set_gemm_config"):
            getattr(other, name).restype = getattr(libs[0], name).restype
            getattr(other, name).argtypes = getattr(libs[0], name).argtypes
        libs[1] = other
        # (the other build may size its workspace differently: take the larger of the two)
        other.dice_moe_workspace_bytes.restype = libs[0].dice_moe_workspace_bytes.restype
        other.dice_moe_workspace_bytes.argtypes = libs[0].dice_moe_workspace_bytes.argtypes
        need = int(other.dice_moe_workspace_bytes(ctypes.byref(desc), x.shape[0]))
        if need > ws.numel() * ws.element_size():
            ws = torch.empty(need, dtype=torch.uint8, device=x.device)
    caller = None
    if call == "modulated":
        B = cfg["samples"]
        g = torch.Generator().manual_seed(1)
        keep = [(torch.randn(B, cfg["D"], generator=g) * 0.3).to(x.dtype).to(dev) for _ in range(3)]
        caller = CallerDesc()
        caller.shift, caller.scale, caller.gate = (ptr(t) for t in keep)
        caller.tokens_per_sample = cfg["tokens"] // B
        caller.ln_eps = 1e-6

    def run(L, n):
        for _ in range(n):
            if caller is None:
                rc = L.dice_moe_forward(ctypes.byref(desc), ptr(x), x.shape[0], 0, None, None, None, ptr(y), None,
                                        None, ptr(ws), ws.numel(), stream_ptr())
            else:
                rc = L.dice_moe_forward_modulated(ctypes.byref(desc), ctypes.byref(caller), ptr(x), x.shape[0], 0,
                                                  None, None, None, ptr(y), None, None, ptr(ws), ws.numel(),
                                                  stream_ptr())
            if rc:
                raise RuntimeError(f"layer call failed with code {rc}")
        torch.cuda.synchronize()

    hooks = (hook_a, hook_b)
    outs = []
    for i in (0, 1):
        libs[i].dice_set_gemm_config(*hooks[i])
        run(libs[i], 10)
        outs.append(y.clone())
    times = ([], [])
    try:
        # (the first two groups are not counted: the first segments after a pause run 2-6 % slow)
        for g, i in enumerate([0, 1, 1, 0] * (groups + 2)):
            libs[i].dice_set_gemm_config(*hooks[i])
            run(libs[i], 2)
            t0 = time.perf_counter()
            run(libs[i], seg)
            if g >= 8:
                times[i].append((time.perf_counter() - t0) / seg * 1e6)
    finally:
        for L in libs:
            L.dice_set_gemm_config(0, 0)
    mean = [statistics.mean(t) for t in times]
    sem = [statistics.stdev(t) / len(t) ** 0.5 for t in times]
    med = [statistics.median(t) for t in times]
    return {"workload": workload_text(cfg, variant, activations), "call": call, "segments": 2 * groups,
            "calls_per_segment": seg,
            "a": {"hook": list(hook_a), "us_per_call": mean[0], "sem": sem[0], "median": med[0],
                  "segments_us": [round(t, 1) for t in times[0]]},
            "b": {"hook": list(hook_b), "lib": lib_b, "us_per_call": mean[1], "sem": sem[1], "median": med[1],
                  "segments_us": [round(t, 1) for t in times[1]]},
            "b_over_a": mean[1] / mean[0], "b_over_a_medians": med[1] / med[0],
            "outputs_bit_identical": bool(torch.equal(outs[0], outs[1]))}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", default="c2", choices=sorted(CONFIGS))
    ap.add_argument("--variant", default="swiglu", choices=["swiglu", "gelu_tanh"])
    ap.add_argument("--activations", default="fp8", choices=["bf16", "fp8", "fp8_blocks"],
                    help="c5 only: bf16 = fp8 weights widened onto the bf16 MFMA; fp8 = rows quantised per token, fp8 MFMA; "
                         "fp8_blocks = fp8 with h quantised inside fc1's epilogue (one power-of-two scale per row and 32 columns)")
    ap.add_argument("--fc1-cfg", type=int, default=0)
    ap.add_argument("--fc2-cfg", type=int, default=0)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-stages", action="store_true", help="skip the per-kernel timing pass")
    ap.add_argument("--no-caller", action="store_true", help="skip the fused-caller (LayerNorm/modulate + residual) pass")
    ap.add_argument("--no-staleness", action="store_true", help="skip the 50-step conditional-communication loop")
    ap.add_argument("--no-lagged", action="store_true", help="skip the step-lagged (displaced / interweaved) pass")
    ap.add_argument("--no-after-idle", action="store_true",
                    help="skip the per-call durations of the first 64 calls after a two-second pause")
    ap.add_argument("--no-sustained", action="store_true",
                    help="skip the sustained pass over eight blocks with distinct weights")
    ap.add_argument("--no-vendor", action="store_true",
                    help="skip the vendor-GEMM reference (torch.matmul on the routed fc1 shape with the same operands)")
    ap.add_argument("--no-configs", action="store_true",
                    help="default run only: skip the short legs of the other configurations")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 256 MiB device copy (a known-size kernel to scale "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings by)")
    ap.add_argument("--ab-hooks", nargs=2, metavar=("A", "B"),
                    help="instead of the benchmark: compare two settings 'fc1,fc2' of the tuning hook on the chosen "
                         "configuration in an A B B A sequence of short segments and print the result")
    ap.add_argument("--ab-lib", default=None, help="with --ab-hooks: setting B runs on this other build of the library")
    ap.add_argument("--ab-tokens", type=int, default=None, help="with --ab-hooks: tokens per call (default: the configuration's)")
    ap.add_argument("--ab-call", default="layer", choices=["layer", "modulated"],
                    help="with --ab-hooks: dice_moe_forward or dice_moe_forward_modulated")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: the layer holds every expert on one MI355X and uses no "
              "collectives; run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs an MI355X; there is no CPU path", file=sys.stderr)
        sys.exit(2)
    from dice_amd import lib
    dev = torch.device("cuda:0")
    if args.ab_hooks:
        a, b = (tuple(int(v) for v in h.split(",")) for h in args.ab_hooks)
        acts = args.activations if CONFIGS[args.config].get("fp8") else "bf16"
        print(json.dumps({"ab": ab_hooks(args.config, args.variant, acts, dev, a, b, args.ab_lib, args.ab_call, args.ab_tokens)}))
        return
    lib.load().dice_set_gemm_config(args.fc1_cfg, args.fc2_cfg)

    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    main_cfg = args.config
    cfg = CONFIGS[main_cfg]
    if cfg.get("staleness"):
        # c4: the step is one layer call of the 50-step loop (full and skip steps as the reference schedules them)
        x = make_input(cfg, dev)
        loop = time_staleness(cfg, args.variant, dev, x)
        ms = loop["high"]["ms_per_step"]
        out = {"metric": "MoE-layer tokens/s, DiT-XL/2-MoE staleness loop (high) 8192 tok bf16",
               "value": cfg["tokens"] / (ms * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": 50, "warmup": 50,
               "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
               "data": "synthetic", "config": {"workload": workload_text(cfg, args.variant, "bf16"), "variant": args.variant},
               "staleness_loop_50_steps": loop}
        print(json.dumps(out))
        return

    cfg, blk, x, res = measure(main_cfg, args.variant, args.activations, dev, args.steps, args.warmup,
                               stages=not args.no_stages)
    a8 = bool(cfg.get("fp8")) and args.activations.startswith("fp8")
    metric = {"c1": "MoE-layer tokens/s, DiT-S/2-MoE 1024 tok fp32", "c2": "MoE-layer tokens/s, DiT-XL/2-MoE 8192 tok bf16",
              "c3": "MoE-layer tokens/s, DiT-XL/2-MoE 16384 tok bf16 Zipf router",
              "c5": "MoE-layer tokens/s, DiT-G/2-MoE 8192 tok fp8 experts"}[main_cfg]
    out = {
        "metric": metric,
        "value": res["tokens_per_s"],
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": res["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8" if a8 else cfg["dtype"],
        "data": "synthetic",
        "config": {"workload": res["workload"], "variant": args.variant, "tokens": cfg["tokens"], "hidden": cfg["D"],
                   "experts": cfg["E"], "top_k": cfg["topk"], "fc1_cfg": args.fc1_cfg, "fc2_cfg": args.fc2_cfg},
        "layer_tflops": res["layer_tflops"],
    }
    if cfg["dtype"] == "bf16":
        out["layer_frac_of_bf16_peak"] = res["layer_tflops"] / PEAK_TFLOPS["bf16"]
    for key in ("roofline", "mfma_util_pct_of_peak", "stage_ms", "hbm_stage_gbs", "hbm_stage_frac_of_peak",
                "fp8_launch_frac_of_fp8_peak", "quantiser_gbs"):
        if key in res:
            out[key] = res[key]
    if not args.no_after_idle and main_cfg == "c2":
        # (not part of `value`) the first calls after a pause, one duration per call
        out["ms_per_call_after_2s_idle"] = time_after_idle(blk, x)
    if not args.no_caller:
        out["block_moe_half_ms"] = time_caller(cfg, blk, x, args.steps, args.warmup, (args.fc1_cfg, args.fc2_cfg))
    if not args.no_staleness and main_cfg == "c2":
        # configs[3] on the same block shape (not part of `value`)
        out["staleness_loop_50_steps"] = time_staleness(CONFIGS["c4"], args.variant, dev, x)
    if not args.no_sustained and cfg["dtype"] == "bf16":
        # The reference walks a stack of blocks with distinct weights (not part of `value`): eight blocks of this
        # configuration round-robin for at least a second, the dominant launch timed over that same run.
        sus = time_sustained_cold(cfg, args.variant, dev)
        out["tokens_per_s_sustained_cold"] = sus["tokens_per_s"]
        if "roofline" in out and sus["fc1_ms_per_launch"] > 0:
            ach = out["roofline"]["flop_per_launch"] / (sus["fc1_ms_per_launch"] * 1e-3) / 1e12
            sus["fc1_achieved_tflops"] = ach
            sus["fc1_frac_of_peak"] = ach / out["roofline"]["peak"]
        out["sustained_cold_layers"] = sus
    if not args.no_staleness and main_cfg == "c2":
        # configs[3] with one cache entry per layer over a stack of eight distinct blocks (not part of `value`)
        out["staleness_loop_50_steps_8_layers"] = time_staleness_layers(CONFIGS["c4"], args.variant, dev)
    if not args.no_configs and main_cfg == "c2":
        # (not part of `value`) the same block at the token counts of small sampling batches
        out["ms_per_call_at_other_batch_sizes"] = time_batch_sizes(cfg, args.variant, dev)
    if not args.no_lagged and main_cfg == "c2":
        # the same layer under the reference's step-lagged schedules (not part of `value`)
        out["step_lag_ms_per_layer_call"] = {
            "displaced": time_lagged(cfg, args.variant, dev, x, args.steps, args.warmup, False),
            "interweaved": time_lagged(cfg, args.variant, dev, x, args.steps, args.warmup, True)}
    if not args.no_vendor and cfg["dtype"] == "bf16":
        v = time_vendor_gemm(cfg, blk, x, dev)
        if v:
            out["vendor_gemm_tflops"] = v
        if "roofline" in out:
            # The same launches with every expert weight zero (same instructions, addresses and traffic): how far
            # the board's power limit, which depends on the operand values, sets the time of the dominant kernel.
            zero = make_block(cfg, args.variant, dev, activations=args.activations)
            if zero._packed is None:
                zero.pack_weights()
            for t in (zero._packed.w1, zero._packed.w2, zero._packed.sw1, zero._packed.sw2):
                if t is not None:
                    t.view(torch.uint8).zero_()
            _, zero_fc1_ms = time_layer(zero, x, args.steps, args.warmup)
            out["roofline"]["ms_per_launch_zero_weights"] = zero_fc1_ms
            del zero
    del blk
    if main_cfg == "c2" and not args.no_configs:
        # The other configurations as short legs, each what `--config cN` prints in full.
        legs = {}
        short = max(10, args.steps // 2)
        for name, var, act in (("c1", args.variant, "bf16"), ("c3", args.variant, "bf16"),
                               ("c5", args.variant, "fp8"), ("c5", args.variant, "fp8_blocks"),
                               ("c5", args.variant, "bf16"),
                               ("c2", "gelu_tanh" if args.variant == "swiglu" else "swiglu", "bf16"),
                               ("c5", "gelu_tanh" if args.variant == "swiglu" else "swiglu", "fp8")):
            c, b, xx, r = measure(name, var, act, dev, short, 5, stages=not args.no_stages)
            key = (name + ("_" + var if var != args.variant else "") + ("_w8a16" if c.get("fp8") and act == "bf16" else "")
                   + ("_h_blocks" if act == "fp8_blocks" else ""))
            keep = {q: r[q] for q in ("tokens_per_s", "ms_per_step", "layer_tflops", "workload", "roofline",
                                      "fp8_launch_frac_of_fp8_peak", "quantiser_gbs", "hbm_stage_frac_of_peak") if q in r}
            if "stage_ms" in r:
                keep["stage_ms"] = {q: round(v, 4) for q, v in r["stage_ms"].items()}
            legs[key] = keep
            del b, xx
            torch.cuda.empty_cache()
        out["configs"] = legs
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(cfg, args.variant)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
