"""Benchmark of the MoE layer hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--variant swiglu|gelu_tanh]

A step is one call of the whole layer (router -> dispatch -> grouped expert
MLP + shared expert -> combine) on the DiT-XL/2-MoE block: 8192 tokens,
hidden 1152, 8 experts, top-2, expert intermediate 4608, bf16 with fp32
accumulation, inputs and weights resident in HBM.  Prints ONE JSON line.
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

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0
# Bytes one fc1 launch moves past the L2 (Infinity Cache + HBM), from rocprofv3 --pmc FETCH_SIZE (x2.0, the
# factor a plain 256 MiB copy needs) + WRITE_SIZE (x1.0): profiles/layer_c2_bf16_hbm_traffic.txt.
FC1_HBM_TRAFFIC_BYTES = 0.941e9

N_TOKENS, D, E, TOPK, RATIO = 8192, 1152, 8, 2, 4


def make_block(variant, dev, layer_idx=0, total_layers=1, para_mode=None):
    """Seeded synthetic weights: router N(0, 0.02), experts Xavier-uniform."""
    from dice_amd import ParaMode, SparseMoeBlock
    # swiglu: the reference's shared expert (one SwiGLU MLP of width 2D, models.py:292-296);
    # gelu_tanh: two always-on experts of the routed shape = one MLP of width 2*4D.
    n_shared = 2 if variant == "swiglu" else 2 * RATIO
    torch.manual_seed(layer_idx)
    blk = SparseMoeBlock(D, RATIO, E, TOPK, pretraining_tp=1, layer_idx=layer_idx, total_layers=total_layers,
                         para_mode=para_mode or ParaMode(), variant=variant, n_shared_experts=n_shared)
    for m in blk.modules():
        if isinstance(m, torch.nn.Linear):
            torch.nn.init.xavier_uniform_(m.weight)
            if m.bias is not None:
                torch.nn.init.zeros_(m.bias)
    torch.nn.init.normal_(blk.gate.weight, std=0.02)
    return blk.to(device=dev, dtype=torch.bfloat16).eval()


def layer_flops(variant):
    slots = N_TOKENS * TOPK
    inter = RATIO * D
    if variant == "swiglu":
        fc1 = 2.0 * slots * (2 * inter) * D
        fc2 = 2.0 * slots * D * inter
        s1 = 2.0 * N_TOKENS * (2 * 2 * D) * D
        s2 = 2.0 * N_TOKENS * D * (2 * D)
    else:
        fc1 = 2.0 * slots * inter * D
        fc2 = 2.0 * slots * D * inter
        s1 = 2.0 * N_TOKENS * (2 * inter) * D
        s2 = 2.0 * N_TOKENS * D * (2 * inter)
    return {"fc1": fc1, "fc2": fc2, "shared_fc1": s1, "shared_fc2": s2}


def time_layer(blk, x, steps, warmup):
    """Seconds per step over `steps` back-to-back layer calls, and the mean duration
    (ms) of the dominant launch (the fc1 expert GEMM) over the SAME calls: the library
    brackets that one launch with two HIP events per call on the stream it launches on
    (event rings of 64 calls, read without stopping the clock in between)."""
    import ctypes
    from dice_amd.lib import check, load
    lib = load()
    n = lib.dice_profile_stage_count()
    names = [lib.dice_profile_stage_name(i).decode() for i in range(n)]
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


def time_stages(blk, x, steps):
    """Mean duration of every launch of the layer in ms, from the library's own
    stage timers: HIP events recorded between the launches of dice_moe_forward
    on the stream it launches on (torch's current stream)."""
    import ctypes
    from dice_amd.lib import check, load
    lib = load()
    check(lib.dice_profile_enable(1))
    n = lib.dice_profile_stage_count()
    names = [lib.dice_profile_stage_name(i).decode() for i in range(n)]
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


def time_staleness(variant, dev, x, sample_steps=50):
    """Configuration 4: the conditional-communication loop of the reference sampler
    (diffusion/rectified_flow.py:83-105) on this layer: 50 steps counted down, the first a
    full step, then skip steps (half of the routed slots recomputed, the other half read
    from the per-layer cache) alternating with full steps that refill the cache; x drifts
    by 0.05 N(0,1) per step.  Returns ms per step for each strategy and per step kind."""
    from dice_amd import ParaMode, diep
    blk = make_block(variant, dev, 0, 1, ParaMode(ep=True))
    xv = x.view(1, N_TOKENS, D)
    g = torch.Generator(device=dev).manual_seed(4)
    noise = [0.05 * torch.randn(xv.shape, generator=g, device=dev, dtype=torch.float32) for _ in range(4)]
    out = {}
    try:
        for mode in ("high", "low", "rand"):
            diep.ep_cache_init(cache_capacity=1, noskip_step=2, skip_mode=mode)
            diep.ep_set_rand_mask(None)
            kinds = {"full": [0.0, 0], "skip": [0.0, 0]}
            total = 0.0
            for rep in range(2):            # first repetition warms up
                xt = xv.clone()
                for i in range(sample_steps, 0, -1):
                    diep.ep_set_step(i)
                    if diep.ep_forced_sync(i, sample_steps):
                        diep.ep_cache_clear()
                    kind = "skip" if diep.ep_skip_now(0) else "full"
                    torch.cuda.synchronize()
                    t0 = time.perf_counter()
                    blk(xt)
                    torch.cuda.synchronize()
                    dt = time.perf_counter() - t0
                    if rep == 1:
                        kinds[kind][0] += dt
                        kinds[kind][1] += 1
                        total += dt
                    xt = (xt.float() + noise[i % 4]).to(xt.dtype)
            out[mode] = {"ms_per_step": total / sample_steps * 1e3,
                         "full_put_step_ms": kinds["full"][0] / max(1, kinds["full"][1]) * 1e3,
                         "skip_step_ms": kinds["skip"][0] / max(1, kinds["skip"][1]) * 1e3,
                         "full_steps": kinds["full"][1], "skip_steps": kinds["skip"][1]}
    finally:
        diep.ep_cache_init(cache_capacity=1, noskip_step=1)
    return out


def time_lagged(variant, dev, x, steps, warmup, pipeline):
    """ms per layer call of the step-lagged modes on the same block shape: two
    layers, a forced-sync first step, then `steps` lagged steps (displaced: each
    layer two steps behind itself; interweaved: each layer runs the other one's
    experts and is one step behind).  Includes the per-call copy of the layer
    input and the allocation of the cached entry on the host side."""
    from dice_amd import ParaMode, diep
    pm = ParaMode(ep=True, ep_async=True, ep_async_mode="all")
    blks = [make_block(variant, dev, l, 2, pm) for l in range(2)]
    diep.ep_cache_init(cache_capacity=2, async_pipeline=pipeline, selective_async_strategy="all")
    diep.use_latest_expert_weights(True)
    xv = x.view(1, N_TOKENS, D)
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


def time_caller(blk, x, steps, warmup):
    """The MoE line of the reference's DiTBlock.forward, x + gate * moe(modulate(norm2(x))),
    on 32 samples x 256 tokens: ms per call with the prologue / epilogue inside the library,
    with them as torch eager ops around the plain layer call (what the reference's DiTBlock
    does), and the prologue kernel alone with its share of the 8 TB/s HBM peak."""
    import torch.nn.functional as F
    from dice_amd import ops
    B, T = 32, N_TOKENS // 32
    g = torch.Generator().manual_seed(1)
    xs = x.view(B, T, D)
    shift, scale, gate = ((torch.randn(B, D, generator=g) * 0.3).bfloat16().to(x.device) for _ in range(3))
    out = torch.empty_like(xs)

    def fused():
        blk.forward_modulated(xs, shift, scale, gate, out=out)

    def eager():
        h = F.layer_norm(xs, (D,), None, None, 1e-6) * (1 + scale.unsqueeze(1)) + shift.unsqueeze(1)
        return xs + gate.unsqueeze(1) * blk(h)

    def prologue():
        ops.ln_modulate(xs, shift, scale)

    res = {}
    for name, fn in (("fused", fused), ("eager_caller", eager), ("ln_modulate_kernel", prologue)):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        res[name] = (time.perf_counter() - t0) / steps * 1e3
    res["ln_modulate_frac_of_hbm_peak"] = 2 * N_TOKENS * D * 2 / (res["ln_modulate_kernel"] * 1e-3) / 1e9 / PEAK_HBM_GBS
    return res


def cpu_baseline(variant, budget_s=20.0):
    """The oracle (a torch restatement of the reference block) timed on the
    host cores on a bounded token sample of the same workload."""
    from oracle import dice_oracle as O
    cores = min(16, os.cpu_count() or 1)
    torch.set_num_threads(cores)
    n_shared = 2 if variant == "swiglu" else 2 * RATIO
    p = O.make_block_params(D, E, TOPK, RATIO, n_shared, seed=0, dtype=torch.bfloat16, variant=variant)
    g = torch.Generator().manual_seed(1)
    probe = torch.randn(1, 256, D, generator=g).bfloat16()
    O.sparse_moe_block_forward(p, probe)
    t0 = time.perf_counter()
    O.sparse_moe_block_forward(p, probe)
    per_tok = (time.perf_counter() - t0) / 256
    sample = int(min(N_TOKENS, max(256, (budget_s / 4) / max(per_tok, 1e-9))))
    sample = max(256, sample // 256 * 256)
    xs = torch.randn(1, sample, D, generator=g).bfloat16()
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
    return {"value": sample / t, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"{sample} of {N_TOKENS} tokens per call (tokens are independent), bf16 torch oracle of the "
                      f"reference block, median of {reps} calls after 2 warm-ups, {t:.3f} s each, "
                      f"{sum(times):.1f} s of CPU work"}


def time_vendor_gemm(blk, x, dev):
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
    a = x.repeat(TOPK, 1)
    w1 = blk._packed.w1[0]
    big = torch.randn(8192, 8192, device=dev).to(x.dtype)
    return {"routed_fc1_shape_%dx%dx%d" % (a.shape[0], w1.shape[0], a.shape[1]): run(a, w1),
            "8192x8192x8192_randn": run(big, big)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--variant", default="swiglu", choices=["swiglu", "gelu_tanh"])
    ap.add_argument("--fc1-cfg", type=int, default=0)
    ap.add_argument("--fc2-cfg", type=int, default=0)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-stages", action="store_true", help="skip the per-kernel timing pass")
    ap.add_argument("--no-caller", action="store_true", help="skip the fused-caller (LayerNorm/modulate + residual) pass")
    ap.add_argument("--no-staleness", action="store_true", help="skip the 50-step conditional-communication loop")
    ap.add_argument("--no-lagged", action="store_true", help="skip the step-lagged (displaced / interweaved) pass")
    ap.add_argument("--no-vendor", action="store_true",
                    help="skip the vendor-GEMM reference (torch.matmul on the routed fc1 shape with the same operands)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 256 MiB device copy (a known-size kernel to scale "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings by)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: the layer holds every expert on one MI355X and uses no "
              "collectives; run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs an MI355X; there is no CPU path", file=sys.stderr)
        sys.exit(2)
    from dice_amd import lib
    lib.load().dice_set_gemm_config(args.fc1_cfg, args.fc2_cfg)
    dev = torch.device("cuda:0")
    blk = make_block(args.variant, dev)
    x = torch.randn(N_TOKENS, D, generator=torch.Generator().manual_seed(0)).bfloat16().to(dev)

    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    sec, fc1_ms = time_layer(blk, x, args.steps, args.warmup)
    flops = layer_flops(args.variant)
    total_flops = sum(flops.values())
    out = {
        "metric": "MoE-layer tokens/s, DiT-XL/2-MoE 8192 tok bf16",
        "value": N_TOKENS / sec,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": sec * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"DiT-XL/2-MoE block (configs[1]): 8192 tokens x 1152, 8 experts top-2, "
                        f"expert 1152->4608->1152 {args.variant}, shared expert "
                        f"{'1152->2304->1152 (reference)' if args.variant == 'swiglu' else '2 x (1152->4608->1152)'}, "
                        f"bf16 in/out, fp32 accumulate",
            "variant": args.variant,
            "tokens": N_TOKENS, "hidden": D, "experts": E, "top_k": TOPK,
            "fc1_cfg": args.fc1_cfg, "fc2_cfg": args.fc2_cfg,
        },
        "layer_tflops": total_flops / sec / 1e12,
        "layer_frac_of_bf16_peak": total_flops / sec / 1e12 / PEAK_BF16_TFLOPS,
    }
    # Dominant kernel: the persistent fc1 launch (routed experts + shared expert, activation
    # fused), timed inside the timed region above.
    dom_flops = flops["fc1"] + flops["shared_fc1"]
    ach = dom_flops / (fc1_ms * 1e-3) / 1e12
    swiglu = args.variant == "swiglu"
    out["roofline"] = {"bound": "mfma",
                       "kernel": "gemm_persist_kernel4<fc1 %s> (routed + shared expert fc1, activation fused)"
                                 % ("SwiGLU" if swiglu else "GELU-tanh, biased"),
                       "achieved": ach, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                       "frac": ach / PEAK_BF16_TFLOPS,
                       # counters were collected for the reference (SwiGLU) expert only
                       "traffic": FC1_HBM_TRAFFIC_BYTES if swiglu else None,
                       "flop_per_launch": dom_flops, "ms_per_launch": fc1_ms}
    if not args.no_stages:
        # every launch of the layer, in a second pass of back-to-back calls
        st = time_stages(blk, x, max(5, args.steps))
        gemm_ms = st["moe.mlp.fc1"] + st["moe.mlp.fc2"]
        out["mfma_util_pct_of_peak"] = 100.0 * total_flops / (gemm_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS
        out["stage_ms"] = st
        bf = 2
        slots = N_TOKENS * TOPK
        # (the row gather is part of the fc1 kernel's loads on this path: "moe.gather" only
        # shows the timer's own overhead)
        hbm = {"moe.gate": N_TOKENS * D * bf + slots * 8,
               "moe.dispatch": slots * 12,
               "moe.combine": (slots * D + 2 * N_TOKENS * D) * bf + slots * 8}
        out["hbm_stage_gbs"] = {s: hbm[s] / (st[s] * 1e-3) / 1e9 for s in hbm}
        out["hbm_stage_frac_of_peak"] = {s: v / PEAK_HBM_GBS for s, v in out["hbm_stage_gbs"].items()}
    if not args.no_caller:
        out["block_moe_half_ms"] = time_caller(blk, x, args.steps, args.warmup)
    if not args.no_staleness:
        # configs[3]: the 50-step conditional-communication loop (synchronised per step: host-visible latency)
        out["staleness_loop_50_steps"] = time_staleness(args.variant, dev, x)
    if not args.no_lagged:
        # the same layer under the reference's step-lagged schedules (not part of `value`)
        out["step_lag_ms_per_layer_call"] = {
            "displaced": time_lagged(args.variant, dev, x, args.steps, args.warmup, False),
            "interweaved": time_lagged(args.variant, dev, x, args.steps, args.warmup, True)}
    if not args.no_vendor:
        out["vendor_gemm_tflops"] = time_vendor_gemm(blk, x, dev)
        # The same launches with every expert weight zero (same instructions, addresses and traffic): how far the
        # board's power limit, which depends on the operand values, sets the time of the dominant kernel.
        zero = make_block(args.variant, dev)
        zero.pack_weights()
        for t in (zero._packed.w1, zero._packed.w2, zero._packed.sw1, zero._packed.sw2):
            if t is not None:
                t.zero_()
        _, zero_fc1_ms = time_layer(zero, x, args.steps, args.warmup)
        out["roofline"]["ms_per_launch_zero_weights"] = zero_fc1_ms
        del zero
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(args.variant)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
