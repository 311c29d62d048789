"""Staleness control surface of the reference on one GPU: module-level state
with the reference's function names (expertpara/diep.py:36-176), its per-layer
skip cache (expertpara/ep_cache.py:188-235) and the dispatch / combine caches
of its asynchronous expert parallelism (expertpara/diep.py:17-28,184-289;
expertpara/ep_cache.py:62-186).

On one GPU every all-to-all of the reference is a copy, so what remains of
"displaced" and "interweaved" parallelism is the step lag itself: which earlier
call's routing the experts run on and which earlier call's result is returned.
That bookkeeping is host-side and tiny and lives here; the data path (recompute
only the retained slot of every token, blend with the cached expert output,
write the cache on a full step, run the experts on a stale entry, combine an
older one) runs inside ``dice_moe_forward`` / ``dice_moe_forward_lagged``.
"""
from __future__ import annotations

from typing import List, Optional

import torch

_step = 0
_forced_sync = False
_async_pipeline = False
_selective_async_strategy: Optional[str] = None
_use_latest_expert_weights: Optional[bool] = None
max_mem = -1
_noskip_interval = 1
_enable_skip = False
_skip_mode: Optional[str] = None
_rand_mask: Optional[torch.Tensor] = None
_mask_cache = {}      # (mode, length) -> CPU bool mask
_device_masks = {}    # (id of the CPU mask, device) -> (CPU mask, its uint8 device copy)


class EPSkipCache:
    """One tensor per layer; ``get`` empties the entry so a stale row can never
    be consumed twice (reference ep_cache.py:215-220)."""

    def __init__(self, capacity: int):
        self.capacity = capacity
        self.cache: List[Optional[torch.Tensor]] = [None] * capacity

    def clear(self):
        self.cache = [None] * self.capacity

    def put(self, key: int, tensor: torch.Tensor):
        assert isinstance(key, int)
        assert isinstance(tensor, torch.Tensor)
        self.cache[key] = tensor

    def get(self, key: int):
        assert isinstance(key, int)
        value = self.cache[key]
        self.cache[key] = None
        return value

    def contains(self, key: int) -> bool:
        assert isinstance(key, int)
        return self.cache[key] is not None

    def tensors_size(self) -> int:
        return sum(x.element_size() * x.numel() for x in self.cache if isinstance(x, torch.Tensor))


_diep_cache_skip = EPSkipCache(0)


class LagEntry:
    """One layer call's routing and what it refers to: the value tuple of the
    reference's dispatch cache (diep.py:17-21) and, once ``rows`` is filled, of
    its combine cache (diep.py:23-27).  ``x`` is a private copy of the layer
    input (the reference's ``grouped_dup_inp`` is one too), ``rows`` the
    grouped, unweighted expert outputs, ``dropped`` says the dispatch left out
    the skipped slot of every token, ``owner`` is the block whose experts the
    entry needs."""

    __slots__ = ("x", "offsets", "perm", "inv_perm", "topk_weight", "rows", "max_rows", "dropped", "owner",
                 "_rows_buf")

    def __init__(self, x, n_experts: int, top_k: int, dropped: bool, owner=None, copy_x: bool = True):
        n = x.shape[0]
        dev = x.device
        self.x = torch.empty_like(x) if copy_x else x
        self.offsets = torch.empty(n_experts + 1, dtype=torch.int32, device=dev)
        self.perm = torch.empty(n * top_k, dtype=torch.int32, device=dev)
        self.inv_perm = torch.empty(n * top_k, dtype=torch.int32, device=dev)
        self.topk_weight = torch.empty(n * top_k, dtype=torch.float32, device=dev)
        self.rows = None
        self._rows_buf = None
        self.max_rows = n * (top_k - 1) if dropped else n * top_k
        self.dropped = dropped
        self.owner = owner

    @classmethod
    def from_tables(cls, x, offsets, perm, inv_perm, topk_weight, top_k: int, dropped: bool, owner=None):
        """An entry around routing tables that already exist (``x`` is kept as
        given: pass a copy if the caller may change it)."""
        e = cls.__new__(cls)
        n = x.shape[0]
        e.x, e.offsets, e.perm, e.inv_perm, e.topk_weight = x, offsets, perm, inv_perm, topk_weight
        e.rows = None
        e._rows_buf = None
        e.max_rows = n * (top_k - 1) if dropped else n * top_k
        e.dropped = dropped
        e.owner = owner
        return e

    def recycle(self, top_k: int, dropped: bool, owner=None):
        """Makes a retired entry ready for a new call.  The buffers stay;
        ``rows`` reads as None again until the entry has been through the
        experts, its memory is kept aside for ``ensure_rows``."""
        n = self.x.shape[0]
        self.max_rows = n * (top_k - 1) if dropped else n * top_k
        self.dropped = dropped
        self.owner = owner
        if self.rows is not None:
            self._rows_buf, self.rows = self.rows, None

    def ensure_rows(self):
        if self.rows is None:
            buf, self._rows_buf = self._rows_buf, None
            if buf is not None and buf.shape[0] >= max(self.max_rows, 1):
                self.rows = buf
            else:
                self.rows = torch.empty((max(self.max_rows, 1), self.x.shape[-1]), dtype=self.x.dtype,
                                        device=self.x.device)
        return self.rows

    def desc(self):
        from .lib import LagEntryDesc, ptr
        d = LagEntryDesc()
        d.x, d.offsets, d.perm, d.inv_perm = ptr(self.x), ptr(self.offsets), ptr(self.perm), ptr(self.inv_perm)
        d.topk_weight, d.rows, d.max_rows = ptr(self.topk_weight), ptr(self.rows), self.max_rows
        return d

    def tensors(self):
        return [t for t in (self.x, self.offsets, self.perm, self.inv_perm, self.topk_weight, self.rows)
                if isinstance(t, torch.Tensor)]


class All2AllCache:
    """One entry per layer; ``get`` leaves the entry in place (reference
    ep_cache.py:62-118).  There are no handles or send buffers to collect on
    one GPU, so the reference's ``auto_gc`` has nothing to do here."""

    def __init__(self, capacity: int):
        self.capacity = capacity
        self.cache: List[Optional[LagEntry]] = [None] * capacity

    def clear(self):
        self.cache = [None] * self.capacity

    def put(self, key: int, value: LagEntry):
        assert isinstance(key, int) and isinstance(value, LagEntry)
        self.cache[key] = value

    def get(self, key: int) -> LagEntry:
        assert isinstance(key, int)
        assert isinstance(self.cache[key], LagEntry), f"no cached step for layer {key}"
        return self.cache[key]

    def contains(self, key: int) -> bool:
        assert isinstance(key, int)
        return self.cache[key] is not None

    def wait(self):
        """Nothing is in flight on one GPU (reference ep_cache.py:79-85)."""


_diep_cache_dispatch = All2AllCache(0)
_diep_cache_combine = All2AllCache(0)


def ep_cache_init(cache_capacity, auto_gc=False, noskip_step=1, skip_mode=None,
                  async_pipeline=False, selective_async_strategy=None):
    """Reference diep.py:112-158."""
    global _noskip_interval, _enable_skip, _skip_mode, _diep_cache_skip
    global _async_pipeline, _selective_async_strategy, _diep_cache_dispatch, _diep_cache_combine
    assert selective_async_strategy in [None, "shallow", "deep", "interleaved", "all"]
    _selective_async_strategy = selective_async_strategy
    _async_pipeline = async_pipeline
    _noskip_interval = noskip_step
    _enable_skip = noskip_step != 1
    if _enable_skip:
        assert skip_mode is not None
    _skip_mode = skip_mode
    _diep_cache_dispatch = All2AllCache(cache_capacity)
    _diep_cache_combine = All2AllCache(cache_capacity)
    _diep_cache_skip = EPSkipCache(capacity=cache_capacity if _enable_skip else 0)
    _mask_cache.clear()
    _device_masks.clear()


def use_latest_expert_weights(val):
    """Reference ep_fwd.py:12-15: True scales a lagged result with the routing
    weights of the current step, False with those cached beside it."""
    global _use_latest_expert_weights
    assert val in [True, False], "val must be a boolean"
    _use_latest_expert_weights = val


def latest_expert_weights() -> bool:
    return bool(_use_latest_expert_weights)


def diep_force_sync():
    """Reference diep.py:100-103: the calls that follow are synchronous and
    (re)fill the caches; the caller clears them first (rectified_flow.py:100-105)."""
    global _forced_sync
    assert not _forced_sync
    _forced_sync = True


def diep_cancel_sync():
    global _forced_sync
    assert _forced_sync
    _forced_sync = False


def diep_forced_sync() -> bool:
    return _forced_sync


def ep_wait():
    _diep_cache_dispatch.wait()
    _diep_cache_combine.wait()


def layer_is_async(ep_async_mode, layer_idx, total_layers) -> bool:
    """Which layers run step-lagged (reference models.py:328-338)."""
    if ep_async_mode == "shallow":
        return layer_idx < total_layers // 2
    if ep_async_mode == "deep":
        return layer_idx >= total_layers // 2
    if ep_async_mode == "all":
        return True
    if ep_async_mode == "interleaved":
        return layer_idx % 2 == 0
    raise ValueError(f"Invalid ep_async_mode: {ep_async_mode}")


# Per selective-async strategy: (distance to the previous lagged layer, number
# of layers the lagged range wraps over as a fraction of all layers, first
# layer of the range as a fraction of all layers).
_LAG_RANGES = {
    "all": (1, 1.0, 0.0),
    "shallow": (1, 0.5, 0.0),
    "deep": (1, 0.5, 0.5),
    "interleaved": (2, 1.0, 0.0),
}


def _past_layer_key(key):
    """The lagged layer that ran before layer ``key`` (reference
    diep.py:184-194), wrapping from the first lagged layer to the last one of
    the previous step."""
    try:
        back, span_frac, first_frac = _LAG_RANGES[_selective_async_strategy]
    except KeyError:
        raise ValueError(f"Unknown selective async strategy: {_selective_async_strategy}") from None
    layers = _diep_cache_dispatch.capacity
    half = layers // 2
    span = layers if span_frac == 1.0 else half
    first = half if first_frac else 0
    return (key - back) % span + first


def lag_roles(cache_key: int, new_entry: LagEntry):
    """Books ``new_entry`` (this call's routing) into the caches and returns
    ``(work, emit)``: the entry whose experts run in this call and the entry
    this call returns (reference global_dispatch_async diep.py:196-254 and
    global_combine_async :256-289).  On a forced-sync step both are the new
    entry.  Otherwise ``work`` is what the dispatch cache holds for this layer
    (displaced) or for the previous lagged layer (interweaved), and ``emit`` is
    what the combine cache holds for this layer; ``work`` takes the combine
    cache slot of the layer it belongs to."""
    global max_mem
    assert cache_key is not None
    if _forced_sync:
        assert not _diep_cache_dispatch.contains(cache_key)
        assert not _diep_cache_combine.contains(cache_key)
        _diep_cache_dispatch.put(cache_key, new_entry)
        _diep_cache_combine.put(cache_key, new_entry)
        return new_entry, new_entry
    if _async_pipeline:
        past_key = _past_layer_key(cache_key)
        assert _diep_cache_dispatch.contains(past_key)
        assert _diep_cache_combine.contains(cache_key)
    else:
        past_key = cache_key
    work = _diep_cache_dispatch.get(past_key)
    _diep_cache_dispatch.put(cache_key, new_entry)
    emit = _diep_cache_combine.get(cache_key)
    _diep_cache_combine.put(past_key, work)
    max_mem = max(max_mem, ep_cached_tensors_size())
    return work, emit


def lag_entry_cached(entry) -> bool:
    """Whether ``entry`` still sits in the dispatch or the combine cache."""
    return any(e is entry for cache in (_diep_cache_dispatch, _diep_cache_combine) for e in cache.cache)


def ep_get_max_mem():
    return max_mem


def ep_set_step(step):
    global _step
    _step = step


def ep_skip_enabled():
    return _enable_skip


def ep_skip_now(idx):
    """Reference diep.py:61-68."""
    if not _enable_skip or not _diep_cache_skip.contains(idx):
        return False
    return _step % _noskip_interval != 0


def _draw_rand_mask(length):
    """One masked slot per token pair, drawn with the CPU generator exactly as
    the reference draws it (one ``randint(0, 2, (pairs,))`` call, diep.py:80-88),
    so a seeded process gets the reference's mask."""
    pick = torch.randint(0, 2, (length // 2,))
    return torch.stack((pick == 0, pick == 1), dim=1).reshape(-1)


def ep_skip_mask(length):
    """Bool mask over flat slots, one True per token pair (reference
    diep.py:72-90): 'high' = slot 0, 'low' = slot 1, 'rand' = one random slot
    per pair drawn once per process and reused.  A 'rand' mask drawn for
    another length is an error here (the reference fails later, on the shape
    of the indexing it does with it)."""
    global _rand_mask
    if _skip_mode in ("high", "low"):
        key = (_skip_mode, length)
        mask = _mask_cache.get(key)
        if mask is None:
            mask = torch.zeros(length, dtype=torch.bool)
            mask[(0 if _skip_mode == "high" else 1)::2] = True
            _mask_cache[key] = mask
        return mask
    if _skip_mode == "rand":
        if _rand_mask is None:
            _rand_mask = _draw_rand_mask(length)
        if _rand_mask.numel() != length:
            from .lib import DiceError
            raise DiceError(f"the 'rand' skip mask was drawn for {_rand_mask.numel()} slots, this call has {length}: "
                            "the batch changed; install a new mask with ep_set_rand_mask(None)")
        return _rand_mask
    raise ValueError(f"Unknown skip mode: {_skip_mode}")


def mask_on_device(mask, device):
    """``mask`` (a CPU bool tensor from ``ep_skip_mask``) as a uint8 tensor on
    ``device``.  The host policy hands out the same mask object for every layer
    and step, so the copy is made once per (mask, device) and not per layer call."""
    key = (id(mask), str(device))
    hit = _device_masks.get(key)
    if hit is None or hit[0] is not mask:
        if len(_device_masks) > 16:
            _device_masks.clear()
        hit = (mask, mask.to(device).view(torch.uint8))
        _device_masks[key] = hit
    return hit[1]


def ep_skip_mask_on(length, device):
    """``ep_skip_mask(length)`` as a uint8 tensor on ``device``."""
    return mask_on_device(ep_skip_mask(length), device)


def ep_set_rand_mask(mask: Optional[torch.Tensor]):
    """Extension: installs (or clears) the 'rand' mask so runs are reproducible."""
    global _rand_mask
    _rand_mask = mask
    _device_masks.clear()


def ep_cache_clear():
    _diep_cache_dispatch.clear()
    _diep_cache_combine.clear()
    _diep_cache_skip.clear()


def ep_skip_get(key):
    return _diep_cache_skip.get(key)


def ep_skip_put(key, tensor):
    assert isinstance(tensor, torch.Tensor)
    _diep_cache_skip.put(key, tensor)


def ep_skip_cached_tensors_size():
    return _diep_cache_skip.tensors_size()


def ep_all2all_cached_tensors_size():
    """Bytes held by the dispatch and combine caches (reference diep.py:44-48).
    An entry that sits in both caches is counted once; an entry keeps the layer
    input itself ([N, D]) where the reference keeps its k-fold gathered copy."""
    seen, total = set(), 0
    for cache in (_diep_cache_dispatch, _diep_cache_combine):
        for e in cache.cache:
            if e is None:
                continue
            for t in e.tensors():
                if id(t) not in seen:
                    seen.add(id(t))
                    total += t.element_size() * t.numel()
    return total


def ep_cached_tensors_size():
    return ep_all2all_cached_tensors_size() + ep_skip_cached_tensors_size()


def ep_forced_sync(i, sample_steps, ep_async_warm_up=0, strided_sync=0, ep_async_cool_down=0):
    """Step policy of the reference sampler (diffusion/warmup.py:6-26): the
    first step, warm-up steps, every ``strided_sync``-th step and the cool-down
    steps are full steps; the caller clears the caches on them
    (diffusion/rectified_flow.py:100-105)."""
    if i == sample_steps:
        return True
    if ep_async_warm_up < 1 and strided_sync < 1:
        return False
    current_step_rev = sample_steps - i
    if 0 < current_step_rev <= ep_async_warm_up:
        return True
    if strided_sync > 0 and i % strided_sync == 0:
        return True
    if i <= ep_async_cool_down:
        return True
    return False
