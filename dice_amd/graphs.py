"""HIP graphs of the layer for launch-bound sizes.

A call of the layer is six to nine kernel launches and no host work in between
(the C ABI never allocates, synchronises, clears memory with a memset node or
reads a device value on the host), so a caller may record it into a HIP graph.
At the reference's small configurations (DiT-S: 1024 tokens of width 384) the
kernels themselves take a few microseconds each and a call is bound by the
launches; replaying a recorded graph removes them.

``GraphedBlock`` records one call of a ``SparseMoeBlock`` on buffers of a fixed
shape and replays it on new inputs.  The reference has no counterpart: its layer
reads expert counts on the host (models.py:366) and cannot be recorded.
"""
from __future__ import annotations

from typing import Optional

import torch

from .lib import MODE_PLAIN, MODE_PUT, MODE_SKIP, CallerDesc, DiceError, ptr


class GraphedBlock:
    """One recorded call of ``block`` on ``[N, D]`` activations.

    ``mode`` is one of the staleness modes of ``SparseMoeBlock.run``: plain, a
    full step that also writes the skip cache (``MODE_PUT``) or a skip step that
    reads it (``MODE_SKIP``); the mask and the cache are buffers of this object
    (``skip_mask``, ``cache``) that the caller fills between replays.  With
    ``modulated=True`` the recorded call is ``forward_modulated``'s: ``x`` is the
    residual stream and ``shift``, ``scale``, ``gate`` ``[B, D]`` buffers of this
    object.

    ``__call__(x, ...)`` copies its arguments into the recorded buffers on the
    current stream, replays and returns the recorded output buffer ``y`` (valid
    until the next replay).
    """

    def __init__(self, block, n_tokens: int, dtype: Optional[torch.dtype] = None, device=None,
                 mode: int = MODE_PLAIN, modulated: bool = False, samples: int = 1, eps: float = 1e-6,
                 warmup: int = 2):
        if mode not in (MODE_PLAIN, MODE_PUT, MODE_SKIP):
            raise DiceError(f"GraphedBlock: mode {mode}")
        if block.para_mode.ep_async:
            raise DiceError("GraphedBlock records one fixed call; the step-lagged modes change buffers from "
                            "call to call")
        if modulated and (samples < 1 or n_tokens % samples):
            raise DiceError(f"GraphedBlock: {n_tokens} tokens do not split into {samples} samples")
        device = torch.device(device if device is not None else block.gate.weight.device)
        if device.type != "cuda":
            raise DiceError("GraphedBlock needs the block on a GPU")
        dtype = dtype or block.gate.weight.dtype
        d, k = block.embed_dim, block.num_experts_per_tok
        self.block, self.mode, self.modulated, self.eps = block, mode, modulated, eps
        self.x = torch.zeros(n_tokens, d, dtype=dtype, device=device)
        self.y = torch.empty_like(self.x)
        self.skip_mask = None if mode == MODE_PLAIN else torch.zeros(n_tokens * k, dtype=torch.uint8, device=device)
        self.cache = None if mode == MODE_PLAIN else torch.zeros_like(self.x)
        self.shift = self.scale = self.gate = None
        if modulated:
            self.shift, self.scale, self.gate = (torch.zeros(samples, d, dtype=dtype, device=device) for _ in range(3))
        self.graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream(device=device)
        side.wait_stream(torch.cuda.current_stream(device))
        with torch.cuda.stream(side):
            for _ in range(max(1, warmup)):  # packs the weights, sizes the workspace, loads the kernels
                self._call()
        torch.cuda.current_stream(device).wait_stream(side)
        torch.cuda.synchronize(device)
        with torch.cuda.graph(self.graph, stream=side):
            self._call()
        # The recorded launches hold raw addresses: the workspace and the packed weights they name stay
        # alive with this object even if the block later sizes a larger workspace or repacks its weights
        # (a replay then still computes with what was recorded).
        self._recorded_buffers = (block._ws, block._packed)

    def _call(self):
        cache_in = self.cache if self.mode == MODE_SKIP else None
        cache_out = self.cache if self.mode == MODE_PUT else None
        if self.modulated:
            c = CallerDesc()
            c.shift, c.scale, c.gate = ptr(self.shift), ptr(self.scale), ptr(self.gate)
            c.tokens_per_sample = self.x.shape[0] // self.shift.shape[0]
            c.ln_eps = self.eps
            self.block.run(self.x, self.mode, self.skip_mask, cache_in, cache_out, y=self.y, caller=c)
        else:
            self.block.run(self.x, self.mode, self.skip_mask, cache_in, cache_out, y=self.y)

    def replay(self) -> torch.Tensor:
        """Runs the recorded call on whatever the buffers hold."""
        self.graph.replay()
        return self.y

    def __call__(self, x, shift=None, scale=None, gate=None) -> torch.Tensor:
        if x.numel() != self.x.numel() or x.dtype != self.x.dtype:
            raise DiceError(f"GraphedBlock was recorded for {tuple(self.x.shape)} {self.x.dtype}, "
                            f"got {tuple(x.shape)} {x.dtype}")
        self.x.copy_(x.reshape(self.x.shape))
        if self.modulated:
            if shift is None or scale is None or gate is None:
                raise DiceError("GraphedBlock(modulated=True) needs shift, scale and gate")
            self.shift.copy_(shift)
            self.scale.copy_(scale)
            self.gate.copy_(gate)
        return self.replay().view(x.shape)
