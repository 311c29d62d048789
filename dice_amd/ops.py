"""Tensor-level wrappers over the C ABI, one per stage of the layer.

Every function enqueues HIP kernels on torch's current stream and returns
device tensors; none of them synchronises with the host.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import lib as _l
from .lib import DICE_ACT_GELU_TANH, DICE_ACT_SWIGLU, check, dtype_code, load, ptr, stream_ptr

VARIANTS = {"swiglu": DICE_ACT_SWIGLU, "gelu_tanh": DICE_ACT_GELU_TANH}


def gate_topk(x: torch.Tensor, weight: torch.Tensor, top_k: int, norm_topk_prob: bool = False,
              bias: Optional[torch.Tensor] = None, want_logits: bool = False,
              want_int64: bool = False):
    """Router (reference ``MoEGate.forward`` models.py:179-196).

    Returns ``(topk_idx int32 [N,k], topk_weight fp32 [N,k], logits fp32 [N,E] | None,
    topk_idx int64 | None)``; slot 0 is the arg-max."""
    x2 = x.reshape(-1, x.shape[-1])
    n, d = x2.shape
    e = weight.shape[0]
    dev = x2.device
    idx = torch.empty((n, top_k), dtype=torch.int32, device=dev)
    idx64 = torch.empty((n, top_k), dtype=torch.int64, device=dev) if want_int64 else None
    wt = torch.empty((n, top_k), dtype=torch.float32, device=dev)
    logits = torch.empty((n, e), dtype=torch.float32, device=dev) if want_logits else None
    if bias is not None and bias.dtype != torch.float32:
        raise _l.DiceError("router bias must be fp32")
    check(load().dice_gate_topk(ptr(x2), dtype_code(x2.dtype), ptr(weight), dtype_code(weight.dtype),
                                ptr(bias), n, d, e, top_k, int(bool(norm_topk_prob)), ptr(idx),
                                ptr(idx64), ptr(wt), ptr(logits), stream_ptr()))
    return idx, wt, logits, idx64


def dispatch(flat_idx: torch.Tensor, n_experts: int, skip_mask: Optional[torch.Tensor] = None,
             out=None, static_scratch: bool = False):
    """Dispatch tables (reference models.py:365-367, ep_fwd.py:57-76,100-106).

    ``flat_idx`` int32 [S]; ``skip_mask`` uint8/bool [S] marks dropped slots.
    Returns ``(counts [E], offsets [E+1], perm [S], inv_perm [S])`` int32;
    ``out`` may bring these four tensors along.  ``static_scratch`` takes the
    entry point that keeps its histogram table in the library's own device
    array and allocates nothing (given ``out``, neither does this wrapper)."""
    if flat_idx.dtype != torch.int32:
        raise _l.DiceError("dispatch needs int32 expert indices")
    s = flat_idx.numel()
    dev = flat_idx.device
    if out is None:
        counts = torch.empty(n_experts, dtype=torch.int32, device=dev)
        offsets = torch.empty(n_experts + 1, dtype=torch.int32, device=dev)
        perm = torch.empty(s, dtype=torch.int32, device=dev)
        inv_perm = torch.empty(s, dtype=torch.int32, device=dev)
    else:
        counts, offsets, perm, inv_perm = out
        for t, n in ((counts, n_experts), (offsets, n_experts + 1), (perm, s), (inv_perm, s)):
            if t.dtype != torch.int32 or t.numel() < n or t.device != dev:
                raise _l.DiceError("dispatch: an output table is too small, not int32 or on another device")
    if skip_mask is not None:
        if skip_mask.numel() != s or skip_mask.device != dev:
            raise _l.DiceError(f"dispatch: skip mask of {skip_mask.numel()} entries on {skip_mask.device} "
                               f"for {s} slots on {dev}")
        skip_mask = skip_mask.view(torch.uint8) if skip_mask.dtype == torch.bool else skip_mask
    if static_scratch:
        check(load().dice_dispatch_static(ptr(flat_idx), ptr(skip_mask), s, n_experts, ptr(counts),
                                          ptr(offsets), ptr(perm), ptr(inv_perm), stream_ptr()))
        return counts, offsets, perm, inv_perm
    ws_bytes = load().dice_dispatch_workspace_bytes(s, n_experts)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    check(load().dice_dispatch(ptr(flat_idx), ptr(skip_mask), s, n_experts, ptr(counts), ptr(offsets),
                               ptr(perm), ptr(inv_perm), ptr(ws), ws_bytes, stream_ptr()))
    return counts, offsets, perm, inv_perm


def gather_rows(x: torch.Tensor, perm: torch.Tensor, slots_per_token: int, n_rows: int):
    """``out[r] = x[perm[r] // slots_per_token]`` (reference ``_local_dispatch``
    ep_fwd.py:345-347)."""
    out = torch.zeros((n_rows, x.shape[-1]), dtype=x.dtype, device=x.device)
    check(load().dice_gather_rows(ptr(x), dtype_code(x.dtype), ptr(perm), slots_per_token, n_rows,
                                  x.shape[-1], ptr(out), stream_ptr()))
    return out


def grouped_mlp(x: torch.Tensor, perm: Optional[torch.Tensor], slots_per_token: int,
                offsets: torch.Tensor, max_rows: int, w1: torch.Tensor, w2: torch.Tensor,
                variant: str = "swiglu", b1=None, b2=None, w1_scale=None, w2_scale=None,
                scatter_to_slots: bool = False, n_out_rows: Optional[int] = None,
                h: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None):
    """Grouped expert MLP (reference models.py:368-377 with MoeMLP :252-273).

    ``w1`` is ``[E, 2I, D]`` (SwiGLU, rows ``[gate_proj; up_proj]``) or
    ``[E, I, D]`` (GELU); ``w2`` is ``[E, D, I]``.  Returns ``out``: row
    ``perm[r]`` of ``[n_out_rows, D]`` when ``scatter_to_slots`` else row ``r``
    of ``[max_rows, D]``.  Outputs are not scaled by the routing weights."""
    e, d, inter = w2.shape
    if n_out_rows is None:
        n_out_rows = max_rows
    if h is None:
        h = torch.empty((max(max_rows, 1), inter), dtype=x.dtype, device=x.device)
    if out is None:
        out = torch.zeros((n_out_rows, d), dtype=x.dtype, device=x.device)
    check(load().dice_grouped_mlp(
        ptr(x), dtype_code(x.dtype), ptr(perm), slots_per_token, ptr(offsets), e, max_rows, d, inter,
        ptr(w1), ptr(b1), ptr(w2), ptr(b2), ptr(w1_scale), ptr(w2_scale), dtype_code(w1.dtype),
        VARIANTS[variant], ptr(h), ptr(out), int(bool(scatter_to_slots)), stream_ptr()))
    return out


def combine(slot_out: torch.Tensor, topk_weight: torch.Tensor, n_tokens: int, top_k: int,
            inv_perm: Optional[torch.Tensor] = None, shared_out: Optional[torch.Tensor] = None,
            skip_mask: Optional[torch.Tensor] = None, cache_in: Optional[torch.Tensor] = None,
            cache_out: Optional[torch.Tensor] = None):
    """Weighted sum over a token's slots + shared add + cache blend / put
    (reference models.py:377-381,355-357; ep_fwd.py:176-195)."""
    d = slot_out.shape[-1]
    y = torch.empty((n_tokens, d), dtype=slot_out.dtype, device=slot_out.device)
    if skip_mask is not None and skip_mask.dtype == torch.bool:
        skip_mask = skip_mask.view(torch.uint8)
    if topk_weight.dtype != torch.float32:
        raise _l.DiceError("combine needs fp32 routing weights")
    check(load().dice_combine(ptr(slot_out), ptr(inv_perm), ptr(topk_weight), ptr(shared_out),
                              ptr(skip_mask), ptr(cache_in), ptr(cache_out), ptr(y),
                              dtype_code(slot_out.dtype), n_tokens, top_k, d, stream_ptr()))
    return y


def ln_modulate(x: torch.Tensor, shift: torch.Tensor, scale: torch.Tensor, eps: float = 1e-6):
    """``LayerNorm(x) * (1 + scale[:, None]) + shift[:, None]`` without affine
    parameters (reference models.py:75-76,497,519).  ``x [B, T, D]``, ``shift``
    and ``scale`` ``[B, D]``."""
    b, t, d = x.shape
    if shift.shape != (b, d) or scale.shape != (b, d):
        raise _l.DiceError(f"ln_modulate: x {tuple(x.shape)} needs shift and scale [{b}, {d}], "
                           f"got {tuple(shift.shape)} and {tuple(scale.shape)}")
    if shift.dtype != x.dtype or scale.dtype != x.dtype:
        raise _l.DiceError("ln_modulate: shift and scale must have x's dtype")
    x = x.contiguous()
    # Contiguous copies of strided views (chunks of the adaLN output) must stay
    # alive until the launch is enqueued: a temporary dies as soon as its
    # address has been taken and the allocator may hand its block to the next.
    shift_c, scale_c = shift.contiguous(), scale.contiguous()
    out = torch.empty_like(x)
    check(load().dice_ln_modulate(ptr(x), ptr(shift_c), ptr(scale_c), ptr(out),
                                  dtype_code(x.dtype), b * t, d, t, eps, stream_ptr()))
    return out


def quantize_fp8_rowwise(w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-output-channel e4m3fn quantisation of a ``[..., rows, cols]`` weight.
    Returns ``(q float8_e4m3fn same shape, scale fp32 [..., rows])``."""
    cols = w.shape[-1]
    rows = w.numel() // cols
    q = torch.empty(w.shape, dtype=torch.uint8, device=w.device)
    scale = torch.empty(w.shape[:-1], dtype=torch.float32, device=w.device)
    check(load().dice_quantize_fp8_rowwise(ptr(w), dtype_code(w.dtype), rows, cols, ptr(q), ptr(scale),
                                           stream_ptr()))
    return q.view(torch.float8_e4m3fn), scale


def quantize_fp8_act(x: torch.Tensor, perm: Optional[torch.Tensor] = None, slots_per_token: int = 1,
                     n_rows: Optional[torch.Tensor] = None, max_rows: Optional[int] = None
                     ) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-row e4m3fn quantisation of activation rows ``x [*, cols]`` (bf16 /
    fp16), optionally gathered: output row r comes from row
    ``perm[r] // slots_per_token``.  ``n_rows``: int32 device scalar, rows at and
    beyond it are left untouched.  Returns ``(q float8_e4m3fn [max_rows, cols],
    scale fp32 [max_rows])``; untouched rows read as zero bytes / scale 0."""
    cols = x.shape[-1]
    if max_rows is None:
        max_rows = perm.numel() if perm is not None else x.shape[0]
    q = torch.zeros((max_rows, cols), dtype=torch.uint8, device=x.device)
    scale = torch.zeros((max_rows,), dtype=torch.float32, device=x.device)
    check(load().dice_quantize_fp8_act(ptr(x), dtype_code(x.dtype), ptr(perm), slots_per_token, ptr(n_rows),
                                       max_rows, cols, ptr(q), ptr(scale), stream_ptr()))
    return q.view(torch.float8_e4m3fn), scale


def grouped_mlp_a8(x: torch.Tensor, perm: Optional[torch.Tensor], slots_per_token: int,
                   offsets: torch.Tensor, max_rows: int, w1: torch.Tensor, w2: torch.Tensor,
                   w1_scale: torch.Tensor, w2_scale: torch.Tensor, variant: str = "swiglu", b1=None, b2=None,
                   stages: int = 3, h: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                   h_blocks: bool = False):
    """Grouped expert MLP with e4m3 weights AND per-row e4m3 activations on the
    fp8 matrix pipe (``dice_grouped_mlp_a8``).  Returns ``(out [max_rows, D]
    grouped, h [max_rows, I])`` in bf16.  ``h_blocks``: fc1's epilogue writes h
    as e4m3 bytes with one power-of-two scale per row and 32 columns (no
    quantiser launch between the GEMMs); the buffer ``h`` then holds
    ``[max_rows, I]`` bytes followed (from the next multiple of 256 bytes) by
    ``[I / 128, max_rows, 4]`` scale bytes, see ``split_h_blocks``."""
    e, d, inter = w2.shape
    if h is None:
        h = torch.empty((max(max_rows, 1), inter), dtype=x.dtype, device=x.device)
    if out is None:
        out = torch.zeros((max_rows, d), dtype=x.dtype, device=x.device)
    q_rows = torch.empty((max(max_rows, 1), max(d, inter)), dtype=torch.uint8, device=x.device)
    q_scale = torch.empty((max(max_rows, 1),), dtype=torch.float32, device=x.device)
    check(load().dice_grouped_mlp_a8(
        stages, ptr(x), dtype_code(x.dtype), ptr(perm), slots_per_token, ptr(offsets), e, max_rows, d, inter,
        ptr(w1), ptr(b1), ptr(w2), ptr(b2), ptr(w1_scale), ptr(w2_scale), VARIANTS[variant], int(h_blocks),
        ptr(h), ptr(out), ptr(q_rows), ptr(q_scale), stream_ptr()))
    return out, h


def block_scale_order(n_blocks: int) -> torch.Tensor:
    """Where each 32-column block's scale byte sits among its row's: the four scales of 128 columns are one
    dword, stored in the order 0, 2, 1, 3 (``block_scale_pos`` of the library)."""
    cb = torch.arange(n_blocks)
    return (cb & ~3) | ((cb & 1) << 1) | ((cb >> 1) & 1)


def split_h_blocks(h: torch.Tensor, max_rows: int, inter: int):
    """The two parts of an h buffer written with ``h_blocks``: ``(bytes [max_rows, I] uint8 (e4m3),
    exponents [max_rows, I / 32] uint8 in column order)``; a block's values are byte * 2^(exponent - 127)."""
    flat = h.view(torch.uint8).reshape(-1)
    q = flat[:max_rows * inter].view(max_rows, inter)
    start = (max_rows * inter + 255) // 256 * 256
    # stored [I / 128][max_rows][4]: the dwords of a 128-column step are adjacent row after row
    sc = flat[start:start + max_rows * (inter // 32)].view(inter // 128, max_rows, 4).permute(1, 0, 2)
    sc = sc.reshape(max_rows, inter // 32)
    return q, sc[:, block_scale_order(inter // 32).to(sc.device)]


def join_h_blocks(h: torch.Tensor, q: torch.Tensor, exponents: torch.Tensor):
    """Writes e4m3 bytes and per-block exponents (column order) into an h buffer in the layout fc2 reads."""
    max_rows, inter = q.shape
    flat = h.view(torch.uint8).reshape(-1)
    flat[:max_rows * inter] = q.reshape(-1)
    start = (max_rows * inter + 255) // 256 * 256
    stored = torch.empty_like(exponents)
    stored[:, block_scale_order(inter // 32).to(exponents.device)] = exponents
    flat[start:start + stored.numel()] = stored.view(max_rows, inter // 128, 4).permute(1, 0, 2).reshape(-1)
    return h
