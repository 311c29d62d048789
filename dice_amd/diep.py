"""Staleness ("conditional communication") control surface of the reference,
single-GPU part: module-level state with the reference's function names
(expertpara/diep.py:57-98,112-176) and its per-layer skip cache
(expertpara/ep_cache.py:188-235).

The policy is host-side and tiny; the data path (recompute only the retained
slot of every token, blend with the cached expert output, write the cache on a
full step) runs inside ``dice_moe_forward``.
"""
from __future__ import annotations

from typing import List, Optional

import torch

_step = 0
_noskip_interval = 1
_enable_skip = False
_skip_mode: Optional[str] = None
_rand_mask: Optional[torch.Tensor] = None
_mask_cache = {}


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


def ep_cache_init(cache_capacity, auto_gc=False, noskip_step=1, skip_mode=None,
                  async_pipeline=False, selective_async_strategy=None):
    """Reference diep.py:112-158.  ``async_pipeline`` / ``selective_async_strategy``
    configure the cross-GPU all-to-all caches, which do not exist here."""
    global _noskip_interval, _enable_skip, _skip_mode, _diep_cache_skip
    if async_pipeline or selective_async_strategy is not None:
        raise NotImplementedError("async all-to-all staleness needs several GPUs")
    _noskip_interval = noskip_step
    _enable_skip = noskip_step != 1
    if _enable_skip:
        assert skip_mode is not None
    _skip_mode = skip_mode
    _diep_cache_skip = EPSkipCache(capacity=cache_capacity if _enable_skip else 0)
    _mask_cache.clear()


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


def ep_skip_mask(length):
    """Bool mask over flat slots, one True per token pair (reference
    diep.py:72-90): 'high' = slot 0, 'low' = slot 1, 'rand' = one random slot
    per pair drawn once per process and reused."""
    global _rand_mask
    if _skip_mode in ("high", "low"):
        key = (_skip_mode, length)
        if key not in _mask_cache:
            mask = torch.zeros(length, dtype=torch.bool)
            if _skip_mode == "high":
                mask[::2] = True
            else:
                mask[1::2] = True
            _mask_cache[key] = mask
        return _mask_cache[key]
    if _skip_mode == "rand":
        if _rand_mask is None:
            n = length // 2
            bool_tensor = torch.zeros((n, 2), dtype=torch.bool)
            random_indices = torch.randint(0, 2, (n,))
            bool_tensor[torch.arange(n), random_indices] = True
            _rand_mask = bool_tensor.view(-1)
        return _rand_mask
    raise ValueError(f"Unknown skip mode: {_skip_mode}")


def ep_set_rand_mask(mask: Optional[torch.Tensor]):
    """Extension: installs (or clears) the 'rand' mask so runs are reproducible."""
    global _rand_mask
    _rand_mask = mask


def ep_cache_clear():
    _diep_cache_skip.clear()


def ep_skip_get(key):
    return _diep_cache_skip.get(key)


def ep_skip_put(key, tensor):
    assert isinstance(tensor, torch.Tensor)
    _diep_cache_skip.put(key, tensor)


def ep_skip_cached_tensors_size():
    return _diep_cache_skip.tensors_size()


def ep_cached_tensors_size():
    return ep_skip_cached_tensors_size()


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
