"""Shared helpers of the GPU parity tests."""
import contextlib

import torch

from oracle import dice_oracle as O


def rel_l2(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


def check_rows(got: torch.Tensor, want: torch.Tensor, tol: float, what: str = "") -> float:
    """Aggregate relative L2 below ``tol`` AND no single row worse than 5 x tol
    (one bad tile, tail row or token cannot hide inside the norm of thousands
    of good ones).  Returns the aggregate."""
    got, want = got.double().cpu(), want.double().cpu()
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite values"
    agg = float((got - want).norm() / want.norm().clamp_min(1e-30))
    assert agg < tol, f"{what}: rel-L2 {agg:.3e} >= {tol}"
    rows = (got - want).norm(dim=-1) / want.norm(dim=-1).clamp_min(1e-6 * float(want.norm(dim=-1).mean()) + 1e-30)
    worst = int(rows.argmax())
    assert float(rows.max()) < 5 * tol, f"{what}: row {worst} rel err {float(rows.max()):.3e} >= {5 * tol}"
    return agg


def block_from_params(p: O.MoEBlockParams, D, variant="swiglu", dtype=torch.float32, device="cuda",
                      ep=False, layer_idx=0, total_layers=1, para_mode=None, pretraining_tp=1):
    """Builds the product module and loads the oracle's weights through the
    reference's state-dict key layout."""
    from dice_amd import ParaMode, SparseMoeBlock
    E = len(p.experts)
    inter = p.experts[0].gate_proj.shape[0] if variant == "swiglu" else p.experts[0].fc1_w.shape[0]
    n_shared = None
    if p.shared is not None:
        si = p.shared.gate_proj.shape[0] if variant == "swiglu" else p.shared.fc1_w.shape[0]
        n_shared = si // D
    blk = SparseMoeBlock(D, mlp_ratio=inter // D, num_experts=E, num_experts_per_tok=p.top_k,
                         pretraining_tp=pretraining_tp, layer_idx=layer_idx, total_layers=total_layers,
                         para_mode=para_mode if para_mode is not None else ParaMode(ep=ep),
                         variant=variant, n_shared_experts=n_shared)
    sd = {"gate.weight": p.gate_weight}
    def put(prefix, ex):
        if variant == "swiglu":
            sd[prefix + "gate_proj.weight"] = ex.gate_proj
            sd[prefix + "up_proj.weight"] = ex.up_proj
            sd[prefix + "down_proj.weight"] = ex.down_proj
        else:
            sd[prefix + "fc1.weight"], sd[prefix + "fc1.bias"] = ex.fc1_w, ex.fc1_b
            sd[prefix + "fc2.weight"], sd[prefix + "fc2.bias"] = ex.fc2_w, ex.fc2_b
    for e, ex in enumerate(p.experts):
        put(f"experts.{e}.", ex)
    if p.shared is not None:
        put("shared_experts.", p.shared)
    blk.load_state_dict(sd)
    blk = blk.to(device=device, dtype=dtype).eval()
    blk.gate.norm_topk_prob = p.norm_topk_prob
    if p.gate_bias is not None:
        blk.gate.bias = p.gate_bias.float().to(device)
    return blk


@contextlib.contextmanager
def router_own_launch():
    """The modulated layer call with the router as a launch of its own behind the
    prologue kernel (tuning hook, fc1 = 50) instead of inside it."""
    from dice_amd import lib
    lib.load().dice_set_gemm_config(50, 0)
    try:
        yield
    finally:
        lib.load().dice_set_gemm_config(0, 0)


def zipf_bias(E, s=1.2):
    pr = torch.tensor([(e + 1.0) ** -s for e in range(E)])
    pr = pr / pr.sum()
    return pr.log()


@contextlib.contextmanager
def whole_fc2_tiles():
    """Every fc2 tile multiplied whole (tuning hook, fc2 = 50).  By default an fc2
    launch may cut the left-over tiles of a short last turn along k; how many
    depends on the tile count, and the sums of the 16-bit pieces differ from a
    whole tile's in the last bit, so tests that ask for bit-identical outputs
    from calls with different token counts run under this
    (tests/test_gpu_split_turn.py covers the cut itself)."""
    from dice_amd import lib
    lib.load().dice_set_gemm_config(0, 50)
    try:
        yield
    finally:
        lib.load().dice_set_gemm_config(0, 0)
