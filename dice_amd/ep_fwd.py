"""``moe_infer_ep`` of the reference (expertpara/ep_fwd.py:19-197) with its
signature, for callers that bring their own routing: permute -> grouped expert
MLP -> un-permute -> skip-cache blend / put -> scale by the routing weights and
sum a token's slots, assembled from the per-stage entry points of the library.

One GPU holds every expert, so the token-count exchange and both all-to-alls
of the reference (ep_fwd.py:215-342) are absent; with ``async_op`` the call
still returns what the reference returns, the result of an earlier call, through
the caches in ``dice_amd.diep`` (see ``diep.lag_roles``).
"""
from __future__ import annotations

import weakref

import torch

from . import diep, ops
from .diep import use_latest_expert_weights  # noqa: F401  (reference ep_fwd.py:12-15)
from .lib import DiceError

_owners = weakref.WeakKeyDictionary()  # nn.ModuleList of experts -> weakref to its SparseMoeBlock


def register_experts(module_list, block) -> None:
    _owners[module_list] = weakref.ref(block)


def _owner(experts):
    from .moe import SparseMoeBlock
    if isinstance(experts, SparseMoeBlock):
        return experts
    ref = _owners.get(experts)
    blk = ref() if ref is not None else None
    if blk is None:
        raise DiceError("moe_infer_ep: `experts` must be the expert list of a dice_amd.SparseMoeBlock "
                        "(or the block itself): the kernels read its packed weights")
    return blk


@torch.no_grad()
def moe_infer_ep(inp, experts, flat_expert_indices, flat_expert_weights, num_experts_per_tok, async_op,
                 skip_mask=None, skip_now=None, cache_key=None):
    """Arguments as in the reference: ``inp [N, h]``, ``flat_expert_indices
    [N*k]``, ``flat_expert_weights [N*k, 1]`` (or ``[N*k]``), ``skip_mask`` a
    bool mask over the flat slots or None, ``skip_now`` whether this call leaves
    the masked slots out, ``cache_key`` the layer index.  Returns ``[N, h]``."""
    blk = _owner(experts)
    if blk._packed is None:
        blk.pack_weights(blk._fp8)
    p = blk._packed
    n, d = inp.shape
    k = num_experts_per_tok
    n_experts = len(blk.experts)
    partial_skip = skip_mask is not None
    if skip_now:
        assert partial_skip, "skip is not enabled"
        assert k == 2, "only support num_experts_per_tok == 2"
    if flat_expert_indices.numel() != n * k:
        raise DiceError(f"moe_infer_ep: {flat_expert_indices.numel()} expert indices for {n} tokens x {k}")
    x = inp.contiguous()
    idx = flat_expert_indices.to(torch.int32).contiguous()
    mask = None
    if partial_skip:
        if skip_mask.numel() != n * k:
            raise DiceError(f"moe_infer_ep: skip mask of {skip_mask.numel()} entries for {n} tokens x {k}")
        if skip_mask.device != x.device:        # the reference's mask is a CPU tensor (diep.py:72-90)
            skip_mask = diep.mask_on_device(skip_mask, x.device)
        mask = skip_mask.view(torch.uint8) if skip_mask.dtype == torch.bool else skip_mask
    _, offsets, perm, inv_perm = ops.dispatch(idx, n_experts, mask if skip_now else None)
    weights = flat_expert_weights.reshape(-1).float().contiguous()
    new = diep.LagEntry.from_tables(x.clone() if async_op else x, offsets, perm, inv_perm, weights, k,
                                    bool(skip_now), blk)
    if async_op:
        assert cache_key is not None
        work, emit = diep.lag_roles(cache_key, new)
        for entry in (work, emit):
            if entry.x.shape != x.shape or entry.x.dtype != x.dtype:
                raise DiceError("moe_infer_ep: a cached step has another shape: clear the caches and force a "
                                "synchronous step when the batch changes")
    else:
        work = emit = new
    owner = work.owner if work.owner is not None else blk
    # (the block's own arithmetic: the fp8 matrix pipe when it quantises its activations)
    work.rows = owner.routed_experts(work.x, work.perm, work.offsets, work.max_rows, out=work.rows)
    if emit.rows is None:
        raise DiceError("moe_infer_ep: the cached step to return has never been through the experts")
    cache_in = cache_out = None
    if partial_skip:
        if emit.dropped:                                     # reference ep_fwd.py:177-185
            cache_in = diep.ep_skip_get(cache_key)
            if cache_in is None:
                raise DiceError("moe_infer_ep: the skip cache holds nothing for the dropped slots")
            if cache_in.shape != x.shape or cache_in.dtype != x.dtype or cache_in.device != x.device:
                raise DiceError(f"moe_infer_ep: the skip cache holds {tuple(cache_in.shape)} {cache_in.dtype}, this call "
                                f"has {tuple(x.shape)} {x.dtype}: clear the caches when the batch changes")
        else:                                                # :186-188
            cache_out = torch.empty_like(x)
    scale = weights if (diep.latest_expert_weights() or emit is new) else emit.topk_weight
    y = ops.combine(emit.rows, scale.view(n, k), n, k, inv_perm=emit.inv_perm, skip_mask=mask,
                    cache_in=cache_in, cache_out=cache_out)
    if cache_out is not None:
        diep.ep_skip_put(cache_key, cache_out)
    return y
