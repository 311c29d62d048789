"""Reference checkpoints -> MoE blocks of this package.

A DiT-MoE checkpoint of the reference is a flat state dict, optionally wrapped
as ``{"ema": ...}`` or ``{"model": ...}`` by its training script
(download.py:26-33); the MoE layer of transformer block ``b`` owns the keys
(key format: expertpara/etrim.py:44, modules: models.py:280-300, 498-507)

    blocks.{b}.moe.gate.weight                           [E, D]
    blocks.{b}.moe.experts.{e}.gate_proj.weight          [I, D]
    blocks.{b}.moe.experts.{e}.up_proj.weight            [I, D]
    blocks.{b}.moe.experts.{e}.down_proj.weight          [D, I]
    blocks.{b}.moe.shared_experts.{gate,up,down}_proj.weight

This module finds those keys, derives the layer shapes from them, builds
``SparseMoeBlock`` modules and packs their weights into the grouped-GEMM layout
(``w1 [E, 2I, D]`` = rows ``[gate_proj; up_proj]``, ``w2 [E, D, I]``), optionally
quantising the routed experts to fp8.  Everything else in the checkpoint
(attention, embedders, final layer) is left to the caller's model.

``pretraining_tp`` needs nothing here: the reference slices the same weights at
run time (models.py:255-269), the stored tensors do not depend on it.
"""
from __future__ import annotations

import re
from collections import OrderedDict
from typing import Dict, Iterable, List, Mapping, Optional, Tuple

import torch

from .lib import DiceError

_MOE_KEY = re.compile(r"^(?:module\.)?blocks\.(\d+)\.moe\.(.+)$")
_EXPERT_KEY = re.compile(r"^experts\.(\d+)\.(.+)$")


def unwrap_checkpoint(checkpoint: Mapping) -> Mapping[str, torch.Tensor]:
    """The state dict inside a training checkpoint (reference download.py:28-31):
    ``"ema"`` wins over ``"model"``; a bare state dict is returned as is."""
    if "ema" in checkpoint:
        return checkpoint["ema"]
    if "model" in checkpoint:
        return checkpoint["model"]
    return checkpoint


def find_model(model_name: str) -> Mapping[str, torch.Tensor]:
    """Local part of the reference's ``find_model`` (download.py:18-33): loads a
    checkpoint file to host memory and unwraps it.  Tensors only: the file is
    read with ``weights_only=True``.  The reference's download of the dense DiT
    weights (download.py:36-47) has no counterpart."""
    import argparse
    import os
    import pickle
    if not os.path.isfile(model_name):
        raise DiceError(f"Could not find DiT checkpoint at {model_name}")
    # The reference's training script stores its command-line arguments beside
    # the weights ({"model", "ema", "opt", "args": argparse.Namespace},
    # train.py:258-266).  A Namespace is a plain attribute bag whose
    # reconstruction runs no code of the file's choosing, so it is the one class
    # allowed on top of the tensors-only unpickler; anything else in a file is
    # refused, with the name of what was refused.
    try:
        with torch.serialization.safe_globals([argparse.Namespace]):
            checkpoint = torch.load(model_name, map_location="cpu", weights_only=True)
    except pickle.UnpicklingError as e:
        text = str(e)
        m = re.search(r"Unsupported global: GLOBAL (\S+)", text) or re.search(r"Unsupported class (\S+)", text)
        what = m.group(1) if m else text.splitlines()[0][:200]
        raise DiceError(f"{model_name}: not a tensors-only checkpoint ({what}); this loader executes nothing "
                        "from a checkpoint file and accepts tensors, containers, numbers, strings and "
                        "argparse.Namespace only") from None
    if not isinstance(checkpoint, Mapping):
        raise DiceError(f"{model_name}: expected a state dict or a dict wrapping one, got {type(checkpoint).__name__}")
    return unwrap_checkpoint(checkpoint)


def split_moe_state_dict(state_dict: Mapping[str, torch.Tensor]) -> "OrderedDict[int, Dict[str, torch.Tensor]]":
    """``{block index: {key below 'blocks.{b}.moe.': tensor}}`` in block order.
    A ``module.`` prefix (DistributedDataParallel) is accepted."""
    out: Dict[int, Dict[str, torch.Tensor]] = {}
    for key, value in state_dict.items():
        m = _MOE_KEY.match(key)
        if m:
            out.setdefault(int(m.group(1)), {})[m.group(2)] = value
    return OrderedDict(sorted(out.items()))


def moe_layer_shape(sub: Mapping[str, torch.Tensor]) -> dict:
    """Constructor arguments of ``SparseMoeBlock`` read off one layer's tensors."""
    if "gate.weight" not in sub:
        raise DiceError("MoE layer without gate.weight")
    n_experts, embed_dim = sub["gate.weight"].shape
    present = sorted({int(m.group(1)) for m in map(_EXPERT_KEY.match, sub) if m})
    if not present:
        raise DiceError("MoE layer without experts")
    first = f"experts.{present[0]}."
    if first + "gate_proj.weight" in sub:
        variant, inter = "swiglu", sub[first + "gate_proj.weight"].shape[0]
        shared = sub.get("shared_experts.gate_proj.weight")
    elif first + "fc1.weight" in sub:
        variant, inter = "gelu_tanh", sub[first + "fc1.weight"].shape[0]
        shared = sub.get("shared_experts.fc1.weight")
    else:
        raise DiceError(f"unrecognised expert parameters under {first}")
    if inter % embed_dim:
        raise DiceError(f"expert width {inter} is not a multiple of the hidden size {embed_dim}")
    n_shared = None
    if shared is not None:
        if shared.shape[0] % embed_dim:
            raise DiceError(f"shared expert width {shared.shape[0]} is not a multiple of {embed_dim}")
        n_shared = shared.shape[0] // embed_dim
    return {"embed_dim": int(embed_dim), "mlp_ratio": inter // embed_dim, "num_experts": int(n_experts),
            "variant": variant, "n_shared_experts": n_shared, "experts_present": present}


def pack_expert_weights(sub: Mapping[str, torch.Tensor], n_experts: Optional[int] = None,
                        dtype: Optional[torch.dtype] = None, device=None) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(w1 [E, 2I, D], w2 [E, D, I])`` of the SwiGLU routed experts straight
    from one layer's tensors, without building modules: expert ``e`` occupies
    ``w1[e, :I] = gate_proj``, ``w1[e, I:] = up_proj``, ``w2[e] = down_proj``."""
    shape = moe_layer_shape(sub)
    if shape["variant"] != "swiglu":
        raise DiceError("pack_expert_weights packs SwiGLU experts")
    e_total = shape["num_experts"] if n_experts is None else n_experts
    if shape["experts_present"] != list(range(e_total)):
        missing = sorted(set(range(e_total)) - set(shape["experts_present"]))
        raise DiceError(f"experts {missing} are missing (a checkpoint trimmed for expert parallelism "
                        "holds one rank's experts only; this build keeps all experts on one GPU)")
    d, inter = shape["embed_dim"], shape["mlp_ratio"] * shape["embed_dim"]
    ref = sub["experts.0.gate_proj.weight"]
    dtype = dtype or ref.dtype
    device = device or ref.device
    w1 = torch.empty((e_total, 2 * inter, d), dtype=dtype, device=device)
    w2 = torch.empty((e_total, d, inter), dtype=dtype, device=device)
    for e in range(e_total):
        for name, dst in (("gate_proj", w1[e, :inter]), ("up_proj", w1[e, inter:]), ("down_proj", w2[e])):
            src = sub[f"experts.{e}.{name}.weight"]
            if src.shape != dst.shape:
                raise DiceError(f"experts.{e}.{name}.weight has shape {tuple(src.shape)}, expected {tuple(dst.shape)}")
            dst.copy_(src)
    return w1, w2


def build_moe_blocks(state_dict: Mapping[str, torch.Tensor], para_mode=None, num_experts_per_tok: int = 2,
                     pretraining_tp: int = 1, device=None, dtype: Optional[torch.dtype] = None,
                     fp8: bool = False, blocks: Optional[Iterable[int]] = None) -> "OrderedDict[int, torch.nn.Module]":
    """One ``SparseMoeBlock`` per MoE layer of ``state_dict`` (already unwrapped),
    keyed by block index, weights loaded strictly (every parameter must be
    present, nothing below ``blocks.{b}.moe.`` may be left over), moved to
    ``device`` / ``dtype`` and - on a GPU - packed (``fp8`` also quantises the
    routed experts).  ``layer_idx`` / ``total_layers`` are set as the reference's
    ``DiT.__init__`` sets them (models.py:578-594)."""
    from .moe import ParaMode, SparseMoeBlock
    layers = split_moe_state_dict(state_dict)
    if not layers:
        raise DiceError("no 'blocks.{b}.moe.*' keys in the state dict")
    total = max(layers) + 1
    wanted = set(layers) if blocks is None else set(blocks)
    out: "OrderedDict[int, torch.nn.Module]" = OrderedDict()
    for b, sub in layers.items():
        if b not in wanted:
            continue
        shape = moe_layer_shape(sub)
        if shape["experts_present"] != list(range(shape["num_experts"])):
            raise DiceError(f"block {b}: experts {shape['experts_present']} of {shape['num_experts']} present; "
                            "all experts must be in the checkpoint")
        blk = SparseMoeBlock(shape["embed_dim"], shape["mlp_ratio"], shape["num_experts"], num_experts_per_tok,
                             pretraining_tp, layer_idx=b, total_layers=total,
                             para_mode=para_mode if para_mode is not None else ParaMode(),
                             variant=shape["variant"], n_shared_experts=shape["n_shared_experts"])
        blk.load_state_dict(dict(sub), strict=True)
        blk = blk.to(device=device, dtype=dtype).eval()
        if fp8 or (device is not None and torch.device(device).type == "cuda"):
            blk.pack_weights(fp8=fp8)
        out[b] = blk
    return out


def load_moe_state_dict(model: torch.nn.Module, state_dict: Mapping[str, torch.Tensor]) -> List[str]:
    """Loads the MoE layers of ``state_dict`` into the ``SparseMoeBlock``
    modules found in ``model`` at ``blocks.{b}.moe`` (any model whose transformer
    blocks follow the reference's naming).  Returns the MoE keys it consumed."""
    from .moe import SparseMoeBlock
    layers = split_moe_state_dict(state_dict)
    used: List[str] = []
    for name, mod in model.named_modules():
        m = re.match(r"^(?:module\.)?blocks\.(\d+)\.moe$", name)
        if not m or not isinstance(mod, SparseMoeBlock):
            continue
        b = int(m.group(1))
        if b not in layers:
            raise DiceError(f"the checkpoint has no weights for {name}")
        mod.load_state_dict(dict(layers[b]), strict=True)
        used += [f"blocks.{b}.moe.{k}" for k in layers[b]]
    if not used:
        raise DiceError("the model has no SparseMoeBlock at blocks.{b}.moe")
    return used
