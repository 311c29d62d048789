"""Checkpoint handling: the reference's key layout and wrappers -> MoE blocks
and packed grouped-GEMM weights."""
import os

import pytest
import torch

from oracle import dice_oracle as O
from tests.helpers import rel_l2


def _reference_style_state_dict(params_per_block, D, wrap=None, ddp_prefix=False):
    """A flat state dict shaped like a reference DiT-MoE checkpoint: the MoE
    keys of every block (expertpara/etrim.py:44) among other parameters of the
    model, optionally wrapped as train.py wraps it (download.py:28-31)."""
    sd = {"x_embedder.proj.weight": torch.zeros(D, 4, 2, 2), "pos_embed": torch.zeros(1, 16, D),
          "final_layer.linear.weight": torch.zeros(32, D)}
    for b, p in enumerate(params_per_block):
        pre = f"blocks.{b}."
        sd[pre + "attn.qkv.weight"] = torch.zeros(3 * D, D)
        sd[pre + "adaLN_modulation.1.weight"] = torch.zeros(6 * D, D)
        sd[pre + "moe.gate.weight"] = p.gate_weight
        for e, ex in enumerate(p.experts):
            sd[pre + f"moe.experts.{e}.gate_proj.weight"] = ex.gate_proj
            sd[pre + f"moe.experts.{e}.up_proj.weight"] = ex.up_proj
            sd[pre + f"moe.experts.{e}.down_proj.weight"] = ex.down_proj
        sd[pre + "moe.shared_experts.gate_proj.weight"] = p.shared.gate_proj
        sd[pre + "moe.shared_experts.up_proj.weight"] = p.shared.up_proj
        sd[pre + "moe.shared_experts.down_proj.weight"] = p.shared.down_proj
    if ddp_prefix:
        sd = {"module." + k: v for k, v in sd.items()}
    return {wrap: sd, "opt": {"lr": 1e-4}} if wrap else sd


def test_unwrap_prefers_ema_then_model():
    from dice_amd import checkpoint as C
    a, b = {"w": torch.zeros(1)}, {"w": torch.ones(1)}
    assert C.unwrap_checkpoint({"ema": a, "model": b}) is a
    assert C.unwrap_checkpoint({"model": b, "opt": {}}) is b
    assert C.unwrap_checkpoint(a) is a


def test_split_shapes_and_packing_layout():
    from dice_amd import checkpoint as C
    D, E = 64, 4
    params = [O.make_block_params(D, E, 2, 4, 2, seed=s) for s in (1, 2, 3)]
    sd = _reference_style_state_dict(params, D, ddp_prefix=True)
    layers = C.split_moe_state_dict(sd)
    assert list(layers) == [0, 1, 2]
    assert len(layers[1]) == 1 + 3 * E + 3                     # nothing but the MoE keys
    shape = C.moe_layer_shape(layers[2])
    assert shape == {"embed_dim": D, "mlp_ratio": 4, "num_experts": E, "variant": "swiglu",
                     "n_shared_experts": 2, "experts_present": list(range(E))}
    w1, w2 = C.pack_expert_weights(layers[2])
    assert w1.shape == (E, 2 * 4 * D, D) and w2.shape == (E, D, 4 * D)
    for e, ex in enumerate(params[2].experts):
        assert torch.equal(w1[e, :4 * D], ex.gate_proj)        # gate rows first,
        assert torch.equal(w1[e, 4 * D:], ex.up_proj)          # then up rows
        assert torch.equal(w2[e], ex.down_proj)


def test_trimmed_or_damaged_checkpoints_are_refused():
    from dice_amd import DiceError, checkpoint as C
    D, E = 64, 4
    sd = _reference_style_state_dict([O.make_block_params(D, E, 2, 4, 2, seed=1)], D)
    # a checkpoint trimmed for expert parallelism (etrim.py:36-60) keeps every W-th expert
    trimmed = {k: v for k, v in sd.items() if ".experts.1." not in k and ".experts.3." not in k}
    with pytest.raises(DiceError, match="missing"):
        C.pack_expert_weights(C.split_moe_state_dict(trimmed)[0])
    with pytest.raises(DiceError):
        C.build_moe_blocks(trimmed)
    with pytest.raises(DiceError, match="no 'blocks"):
        C.build_moe_blocks({"pos_embed": torch.zeros(1)})
    bad = dict(sd)
    bad["blocks.0.moe.experts.2.up_proj.weight"] = torch.zeros(8, D)
    with pytest.raises(DiceError, match="shape"):
        C.pack_expert_weights(C.split_moe_state_dict(bad)[0])
    extra = dict(sd)
    extra["blocks.0.moe.experts.0.bogus"] = torch.zeros(1)
    with pytest.raises(RuntimeError):
        C.build_moe_blocks(extra)                              # strict load: unexpected key


def test_build_blocks_from_file_on_cpu(tmp_path):
    """find_model -> build_moe_blocks on the host: modules carry the reference's
    state-dict keys and values; indices follow the checkpoint's block numbers."""
    from dice_amd import checkpoint as C
    D, E = 64, 4
    params = [O.make_block_params(D, E, 2, 4, 2, seed=s) for s in (5, 6)]
    path = os.path.join(tmp_path, "dit_moe.pt")
    torch.save(_reference_style_state_dict(params, D, wrap="ema"), path)
    sd = C.find_model(path)
    blocks = C.build_moe_blocks(sd, pretraining_tp=2)
    assert list(blocks) == [0, 1]
    for b, blk in blocks.items():
        assert blk.layer_idx == b and blk.total_layers == 2 and not blk.training
        got = blk.state_dict()
        want = C.split_moe_state_dict(sd)[b]
        assert set(got) == set(want)
        assert all(torch.equal(got[k], want[k]) for k in want)
    with pytest.raises(Exception):
        C.find_model(os.path.join(tmp_path, "absent.pt"))


def test_train_script_checkpoint_opens_weights_only(tmp_path):
    """The file the reference's train.py writes (train.py:258-266): model, ema,
    optimizer state and ``"args": argparse.Namespace``.  It must open through
    the tensors-only loader (ema wins), and a file holding any other class must
    be refused by name instead of being unpickled."""
    import argparse
    import collections
    from dice_amd import checkpoint as C
    from dice_amd.lib import DiceError
    D, E = 64, 4
    model = _reference_style_state_dict([O.make_block_params(D, E, 2, 4, 2, seed=7)], D)
    ema = collections.OrderedDict((k, v + 1) for k, v in model.items())
    opt = {"state": {0: {"step": torch.tensor(3.0), "exp_avg": torch.zeros(4), "exp_avg_sq": torch.zeros(4)}},
           "param_groups": [{"lr": 1e-4, "betas": (0.9, 0.999), "eps": 1e-8, "weight_decay": 0, "amsgrad": False,
                             "params": [0]}]}
    args = argparse.Namespace(model="DiT-S/2", image_size=256, num_experts=8, num_experts_per_tok=2,
                              ckpt_every=50000, resume=None, results_dir="results", vae="ema")
    path = os.path.join(tmp_path, "0050000.pt")
    torch.save({"model": model, "ema": ema, "opt": opt, "args": args}, path)
    sd = C.find_model(path)
    assert set(sd) == set(ema) and all(torch.equal(sd[k], ema[k]) for k in ema)
    blocks = C.build_moe_blocks(sd)
    assert list(blocks) == [0]

    import fractions
    bad = os.path.join(tmp_path, "bad.pt")
    torch.save({"model": model, "extra": fractions.Fraction(1, 3)}, bad)   # not a tensor, not a Namespace
    with pytest.raises(DiceError, match="Fraction"):
        C.find_model(bad)
    lst = os.path.join(tmp_path, "list.pt")
    torch.save([torch.zeros(2)], lst)
    with pytest.raises(DiceError, match="state dict"):
        C.find_model(lst)


@pytest.mark.gpu
@pytest.mark.parametrize("fp8", [False, True])
def test_blocks_from_checkpoint_match_oracle_on_gpu(tmp_path, fp8):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from dice_amd import checkpoint as C
    dev = torch.device("cuda:0")
    D, E = 256, 8
    params = [O.make_block_params(D, E, 2, 4, 2, seed=s, dtype=torch.bfloat16) for s in (7, 8)]
    path = os.path.join(tmp_path, "dit_moe.pt")
    torch.save(_reference_style_state_dict(params, D, wrap="model"), path)
    blocks = C.build_moe_blocks(C.find_model(path), device=dev, dtype=torch.bfloat16, fp8=fp8)
    x = torch.randn(2, 128, D, generator=torch.Generator().manual_seed(0)).bfloat16()
    for b, blk in blocks.items():
        want, widx, _, logits = O.sparse_moe_block_forward(params[b], x)
        got = blk(x.to(dev)).cpu()
        assert rel_l2(got, want) < (5e-2 if fp8 else 2e-2)
        # the packed storage is what the module's parameters now view
        assert blk.experts[3].up_proj.weight.data_ptr() == blk._packed.w1[3, 4 * D:].data_ptr() or fp8
