"""Drop-in modules for the reference's MoE layer, running on the HIP library.

``MoEGate``, ``MoeMLP`` and ``SparseMoeBlock`` keep the constructor arguments,
sub-module names, parameter names/shapes (state-dict keys) and ``forward``
signatures of the reference classes (models.py:159-217, 240-273, 276-382), so a
checkpoint of the reference loads unchanged and ``DiTBlock`` can call the block
as before.  Only the inference branch exists; there is no training path and no
CPU path - every forward runs the gfx950 kernels.
"""
from __future__ import annotations

import ctypes
import math
from typing import Optional

import torch
import torch.nn as nn

from . import diep, ops
from .lib import (DICE_ACT_GELU_TANH, DICE_ACT_SWIGLU, MODE_PLAIN, MODE_PUT, MODE_SKIP, CallerDesc, DiceError,
                  MoeLayerDesc, check, dtype_code, load, ptr, stream_ptr)


class ParaMode:
    """Value object of the reference (models.py:34-70).  ``ep`` selects the
    ``moe_infer_ep`` data flow (and with it the staleness caches), ``ep_async``
    its step-lagged variants; sequence parallelism needs several GPUs and is
    refused."""

    def __init__(self, ep=False, ep_async=False, sp=False, sp_async=False, num_sampling_steps=None,
                 ep_async_warm_up=None, strided_sync=None, ep_async_cool_down=None,
                 sp_async_warm_up=None, ep_async_mode=None):
        if sp or sp_async:
            raise DiceError("sequence parallelism needs several GPUs and is outside this single-GPU build")
        self.ep = ep
        self.ep_async = ep_async
        if ep_async:
            assert ep
        self.sp = False
        self.sp_async = False
        self.dp = not ep
        self.num_sampling_steps = num_sampling_steps
        self.ep_async_warm_up = ep_async_warm_up
        self.strided_sync = strided_sync
        self.sp_async_warm_up = sp_async_warm_up
        self.ep_async_cool_down = ep_async_cool_down
        self.ep_async_mode = ep_async_mode

    def verbose(self):
        if self.dp:
            return "DP"
        return "DiEP" if self.ep_async else "EP"


class MoEGate(nn.Module):
    """Router (reference models.py:159-217, inference branch)."""

    def __init__(self, embed_dim, num_experts=16, num_experts_per_tok=2, aux_loss_alpha=0.01):
        super().__init__()
        self.top_k = num_experts_per_tok
        self.n_routed_experts = num_experts
        self.scoring_func = "softmax"
        self.alpha = aux_loss_alpha
        self.seq_aux = False
        self.norm_topk_prob = False
        self.gating_dim = embed_dim
        self.weight = nn.Parameter(torch.empty((self.n_routed_experts, self.gating_dim)))
        self.bias = None  # extension: optional fp32 [E] router bias (not in the reference)
        self.reset_parameters()

    def reset_parameters(self) -> None:
        nn.init.kaiming_uniform_(self.weight, a=math.sqrt(5))

    @torch.no_grad()
    def forward(self, hidden_states):
        if self.training:
            raise DiceError("MoEGate: only the inference branch is implemented (call .eval())")
        idx, wt, _, idx64 = ops.gate_topk(hidden_states.contiguous(), self.weight, self.top_k,
                                          self.norm_topk_prob, self.bias, want_int64=True)
        return idx64, wt.to(hidden_states.dtype), None


class MoeMLP(nn.Module):
    """SwiGLU expert (reference models.py:240-273).  ``pretraining_tp`` is
    accepted for interface parity; the slice/cat/sum path it selects in the
    reference is algebraically the same product, which is what runs here."""

    def __init__(self, hidden_size, intermediate_size, pretraining_tp=2):
        super().__init__()
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.gate_proj = nn.Linear(hidden_size, intermediate_size, bias=False)
        self.up_proj = nn.Linear(hidden_size, intermediate_size, bias=False)
        self.down_proj = nn.Linear(intermediate_size, hidden_size, bias=False)
        self.pretraining_tp = pretraining_tp
        self._w1 = self._w2 = None      # [1, 2I, D] / [1, D, I] storage the three parameters are views of
        self._row_range = {}            # (rows, device) -> int32 [0, rows] on the device

    def _apply(self, fn, *args, **kwargs):
        self._w1 = self._w2 = None
        self._row_range = {}
        return super()._apply(fn, *args, **kwargs)

    def adopt_packed(self, w1, w2):
        """Re-points the three parameters at ``w1 [1, 2I, D]`` = rows
        ``[gate_proj; up_proj]`` and ``w2 [1, D, I]`` (slices of a block's
        packed storage, or this expert's own), so the weights exist once and
        ``forward`` needs no concatenation."""
        inter = self.intermediate_size
        self.gate_proj.weight.data = w1[0, :inter]
        self.up_proj.weight.data = w1[0, inter:]
        self.down_proj.weight.data = w2[0]
        self._w1, self._w2 = w1, w2

    def _packed_views(self):
        w = self.gate_proj.weight
        ok = (self._w1 is not None and self._w1.data_ptr() == w.data_ptr() and self._w1.dtype == w.dtype
              and self._w2.data_ptr() == self.down_proj.weight.data_ptr()
              and self.up_proj.weight.data_ptr() == w.data_ptr() + w.numel() * w.element_size())
        if not ok:
            w1 = torch.cat([self.gate_proj.weight, self.up_proj.weight], 0).unsqueeze(0).contiguous()
            w2 = self.down_proj.weight.detach().unsqueeze(0).contiguous()
            self.adopt_packed(w1, w2)
        return self._w1, self._w2

    @torch.no_grad()
    def forward(self, x):
        shape = x.shape
        x2 = x.reshape(-1, shape[-1]).contiguous()
        n = x2.shape[0]
        w1, w2 = self._packed_views()
        key = (n, str(x.device))
        offsets = self._row_range.get(key)
        if offsets is None:
            if len(self._row_range) > 64:
                self._row_range.clear()
            offsets = self._row_range[key] = torch.tensor([0, n], dtype=torch.int32, device=x.device)
        out = ops.grouped_mlp(x2, None, 1, offsets, n, w1, w2, "swiglu")
        return out.view(shape)


class GeluMLP(nn.Module):
    """Two-matrix tanh-GELU expert, ``fc2(gelu_tanh(fc1(x)))`` with biases: the
    MLP the benchmark configurations name (the reference keeps it only as a
    commented-out dense ``Mlp``, models.py:496-497)."""

    def __init__(self, hidden_size, intermediate_size):
        super().__init__()
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.fc1 = nn.Linear(hidden_size, intermediate_size, bias=True)
        self.fc2 = nn.Linear(intermediate_size, hidden_size, bias=True)


class _Packed:
    """Expert weights in the layout the grouped GEMM reads."""

    def __init__(self):
        self.w1 = self.w2 = self.b1 = self.b2 = None
        self.w1_scale = self.w2_scale = None
        self.sw1 = self.sw2 = self.sb1 = self.sb2 = None


class SparseMoeBlock(nn.Module):
    """Mixture-of-experts block with a shared expert (reference models.py:276-382).

    Extra keyword ``variant`` ("swiglu" = reference, "gelu_tanh" = two-matrix
    experts) and ``n_shared_experts`` are extensions with reference defaults.
    """

    def __init__(self, embed_dim, mlp_ratio=4, num_experts=16, num_experts_per_tok=2,
                 pretraining_tp=2, layer_idx=None, total_layers=None, para_mode: ParaMode = None,
                 variant: str = "swiglu", n_shared_experts: Optional[int] = 2):
        super().__init__()
        assert para_mode is not None
        self.num_experts_per_tok = num_experts_per_tok
        self.variant = variant
        inter = int(mlp_ratio * embed_dim)
        if variant == "swiglu":
            mk = lambda i: MoeMLP(embed_dim, i, pretraining_tp)
        elif variant == "gelu_tanh":
            mk = lambda i: GeluMLP(embed_dim, i)
        else:
            raise DiceError(f"unknown expert variant {variant}")
        self.experts = nn.ModuleList([mk(inter) for _ in range(num_experts)])
        from .ep_fwd import register_experts
        register_experts(self.experts, self)  # lets moe_infer_ep(inp, block.experts, ...) find the packed weights
        self.gate = MoEGate(embed_dim, num_experts, num_experts_per_tok)
        self.n_shared_experts = n_shared_experts
        if self.n_shared_experts is not None:
            self.shared_experts = mk(embed_dim * self.n_shared_experts)
        self.layer_idx = layer_idx
        self.total_layers = total_layers
        self.para_mode = para_mode
        self.embed_dim = embed_dim
        self.inter = inter
        self._packed: Optional[_Packed] = None
        self._fp8 = False
        self._act_quant = 0          # fp8 experts: 1 activations quantised per row too (fp8 matrix pipe), 2 h in blocks
        # True: a token's result never depends on what else is in the call (no fc2 tile is cut along k; see
        # dice_moe_layer_t.batch_invariant).  Set it before the first call, or clear ``_desc`` after changing it.
        self.batch_invariant = False
        self._desc = None
        self._ws = None
        self._spare_cache = None     # a skip-cache tensor a skip step has consumed: the next full step writes into it
        self._spare_entries = []     # step-lag entries that have left both caches, for re-use

    # ------------------------------------------------------------------ #
    # weight packing
    # ------------------------------------------------------------------ #
    def _apply(self, fn, *args, **kwargs):
        self._packed = None
        self._desc = None
        self._ws = None
        self._spare_cache = None
        self._spare_entries = []
        return super()._apply(fn, *args, **kwargs)

    def load_state_dict(self, *args, **kwargs):
        self._packed = None
        self._desc = None
        return super().load_state_dict(*args, **kwargs)

    @torch.no_grad()
    def pack_weights(self, fp8: bool = False) -> _Packed:
        """Builds ``w1 [E, 2I, D]`` = rows ``[gate_proj; up_proj]`` and
        ``w2 [E, D, I]`` from the per-expert parameters, then re-points every
        parameter at its slice of the packed storage so the weights exist once.
        ``fp8=True`` additionally quantises the routed experts to e4m3 with
        per-output-channel scales (shared expert stays in the module dtype)."""
        p = _Packed()
        ex = list(self.experts)
        if self.variant == "swiglu":
            p.w1 = torch.stack([torch.cat([e.gate_proj.weight, e.up_proj.weight], 0) for e in ex]).contiguous()
            p.w2 = torch.stack([e.down_proj.weight for e in ex]).contiguous()
            for i, e in enumerate(ex):
                e.adopt_packed(p.w1[i:i + 1], p.w2[i:i + 1])
            if self.n_shared_experts is not None:
                s = self.shared_experts
                p.sw1 = torch.cat([s.gate_proj.weight, s.up_proj.weight], 0).unsqueeze(0).contiguous()
                p.sw2 = s.down_proj.weight.data.unsqueeze(0).contiguous()
                s.adopt_packed(p.sw1, p.sw2)
        else:
            p.w1 = torch.stack([e.fc1.weight for e in ex]).contiguous()
            p.w2 = torch.stack([e.fc2.weight for e in ex]).contiguous()
            p.b1 = torch.stack([e.fc1.bias for e in ex]).float().contiguous()
            p.b2 = torch.stack([e.fc2.bias for e in ex]).float().contiguous()
            for i, e in enumerate(ex):
                e.fc1.weight.data = p.w1[i]
                e.fc2.weight.data = p.w2[i]
            if self.n_shared_experts is not None:
                s = self.shared_experts
                p.sw1 = s.fc1.weight.data.unsqueeze(0).contiguous()
                p.sw2 = s.fc2.weight.data.unsqueeze(0).contiguous()
                p.sb1 = s.fc1.bias.data.float().unsqueeze(0).contiguous()
                p.sb2 = s.fc2.bias.data.float().unsqueeze(0).contiguous()
                s.fc1.weight.data = p.sw1[0]
                s.fc2.weight.data = p.sw2[0]
        if fp8:
            p.w1, p.w1_scale = ops.quantize_fp8_rowwise(p.w1)
            p.w2, p.w2_scale = ops.quantize_fp8_rowwise(p.w2)
        self._packed = p
        self._fp8 = fp8
        self._desc = None
        return p

    def quantize_fp8(self, activations: bool = False, h_blocks: bool = False):
        """Switches the routed experts to e4m3 weights (build-defined path).
        ``activations=True`` also quantises the routed experts' input rows (per
        token, dynamically, in front of each GEMM), so that the products run on
        the fp8 matrix pipe; bf16 blocks whose widths are multiples of 256.
        ``h_blocks=True`` (with ``activations``) has fc1's epilogue quantise h
        itself, with one power-of-two scale per row and 32 columns, instead of
        a quantiser launch with one scale per row."""
        if h_blocks and not activations:
            raise DiceError("quantize_fp8(h_blocks=True) needs activations=True")
        if activations:
            # what the fp8 matrix-pipe kernels and the row quantiser take; refused here, not at the first forward
            for name, width in (("hidden", self.embed_dim), ("expert", self.inter)):
                if width % 256 != 0 or not 768 <= width <= 8192:
                    raise DiceError(f"quantize_fp8(activations=True): {name} width {width} is not a multiple of 256 "
                                    f"between 768 and 8192; use quantize_fp8() (e4m3 weights, 16-bit activations)")
            if next(self.experts.parameters()).dtype != torch.bfloat16:
                raise DiceError("quantize_fp8(activations=True): act_quant (the fp8 matrix-pipe path) takes bf16 "
                                "blocks; use quantize_fp8() (e4m3 weights, 16-bit activations)")
        self.pack_weights(fp8=True)
        self._act_quant = (2 if h_blocks else 1) if activations else 0
        self._desc = None
        return self

    def routed_experts(self, x, perm, offsets, max_rows, out=None):
        """The routed experts' two GEMMs on grouped rows (reference models.py:368-377)
        in the arithmetic this block's layer call uses: e4m3 rows on the fp8 matrix
        pipe when the block quantises its activations, else 16-bit rows.  Returns
        the unweighted expert outputs ``[max_rows, D]`` in grouped order."""
        if self._packed is None:
            self.pack_weights(self._fp8)
        p = self._packed
        k = self.num_experts_per_tok
        if self._act_quant and self._fp8:
            if out is None:
                out = torch.zeros((max(max_rows, 1), self.embed_dim), dtype=x.dtype, device=x.device)
            rows, _ = ops.grouped_mlp_a8(x, perm, k, offsets, max_rows, p.w1, p.w2, p.w1_scale, p.w2_scale,
                                         self.variant, p.b1, p.b2, out=out, h_blocks=self._act_quant == 2)
            return rows
        return ops.grouped_mlp(x, perm, k, offsets, max_rows, p.w1, p.w2, self.variant, p.b1, p.b2,
                               p.w1_scale, p.w2_scale, scatter_to_slots=False, n_out_rows=max(max_rows, 1), out=out)

    def _ensure(self, x: torch.Tensor):
        if self._packed is None:
            self.pack_weights(self._fp8)
        if self._desc is None:
            p = self._packed
            d = MoeLayerDesc()
            d.hidden, d.inter = self.embed_dim, self.inter
            d.n_experts, d.top_k = len(self.experts), self.num_experts_per_tok
            d.act_dtype = dtype_code(x.dtype)
            d.w_dtype = dtype_code(p.w1.dtype)
            d.act_variant = DICE_ACT_SWIGLU if self.variant == "swiglu" else DICE_ACT_GELU_TANH
            d.norm_topk_prob = int(self.gate.norm_topk_prob)
            d.gate_w_dtype = dtype_code(self.gate.weight.dtype)
            d.shared_inter = 0 if p.sw1 is None else p.sw2.shape[-1]
            d.gate_w = ptr(self.gate.weight)
            d.gate_bias = ptr(self.gate.bias)
            d.w1, d.w2 = ptr(p.w1), ptr(p.w2)
            d.b1, d.b2 = ptr(p.b1), ptr(p.b2)
            d.w1_scale, d.w2_scale = ptr(p.w1_scale), ptr(p.w2_scale)
            d.shared_w1, d.shared_w2 = ptr(p.sw1), ptr(p.sw2)
            d.shared_b1, d.shared_b2 = ptr(p.sb1), ptr(p.sb2)
            d.act_quant = int(self._act_quant) if self._fp8 else 0
            d.batch_invariant = int(self.batch_invariant)
            self._desc = d
        return self._desc

    def _workspace(self, desc, n_tokens: int, device):
        need = load().dice_moe_workspace_bytes(ctypes.byref(desc), n_tokens)
        if self._ws is None or self._ws.numel() < need or self._ws.device != device:
            self._ws = torch.empty(need, dtype=torch.uint8, device=device)
        return self._ws

    # ------------------------------------------------------------------ #
    # forward
    # ------------------------------------------------------------------ #
    @torch.no_grad()
    def forward(self, hidden_states):
        """``[B, T, D] -> [B, T, D]`` (reference models.py:302-358)."""
        return self._forward(hidden_states, None)

    @torch.no_grad()
    def forward_modulated(self, x, shift, scale, gate, eps: float = 1e-6, out=None):
        """The MoE line of the reference's ``DiTBlock.forward`` (models.py:519)
        in one call: ``x + gate.unsqueeze(1) * moe(modulate(norm2(x), shift, scale))``
        with ``norm2 = LayerNorm(D, elementwise_affine=False, eps)`` (models.py:497)
        and ``modulate`` of models.py:75-76.  ``x [B, T, D]``; ``shift``, ``scale``,
        ``gate`` ``[B, D]`` (chunks of adaLN_modulation's output are fine: they are
        made contiguous here).  ``out`` may be ``x`` itself."""
        if x.dim() != 3 or shift.shape != (x.shape[0], x.shape[2]):
            raise DiceError("forward_modulated needs x [B, T, D] and shift / scale / gate [B, D]")
        wdt = self.gate.weight.dtype
        if x.dtype != wdt:
            # A residual stream kept in another precision than the layer (fp32 stream, half
            # model under autocast): prologue in the stream's type, layer in its own, epilogue
            # as torch ops in the stream's type.
            h = ops.ln_modulate(x, shift.to(x.dtype), scale.to(x.dtype), eps)
            y = self._forward(h, None).to(x.dtype)
            res = x + gate.to(x.dtype).unsqueeze(1) * y
            if out is not None:
                out.copy_(res)
                return out
            return res
        c = CallerDesc()
        keep = [t.to(x.dtype).contiguous() for t in (shift, scale, gate)]
        c.shift, c.scale, c.gate = (ptr(t) for t in keep)
        c.tokens_per_sample = x.shape[1]
        c.ln_eps = eps
        return self._forward(x, c, out)

    def _forward(self, hidden_states, caller, out=None):
        if self.training:
            raise DiceError("SparseMoeBlock: only the inference branch is implemented (call .eval())")
        orig_shape = hidden_states.shape
        x = hidden_states.reshape(-1, orig_shape[-1]).contiguous()
        wdt = self.gate.weight.dtype
        if x.dtype != wdt:
            # Under autocast the reference's linear layers take their inputs in the module's
            # half type whatever the caller's tensors are (sample_ddp.py:228); without it a
            # mismatch is an error there too.
            if not torch.is_autocast_enabled():
                raise DiceError(f"activations are {x.dtype} but the block's parameters {wdt} "
                                "(cast one of them, or run under torch.autocast)")
            x = x.to(wdt)
            hidden_states = hidden_states.to(wdt)
        if x.shape[0] == 0:  # no tokens: nothing to route, nothing to cache
            return out if out is not None else torch.empty_like(hidden_states)
        y = None if out is None else out.view(-1, orig_shape[-1])
        if not self.para_mode.ep:
            return self.run(x, y=y, caller=caller).view(*orig_shape)
        # reference models.py:325-354
        async_op = bool(self.para_mode.ep_async) and diep.layer_is_async(
            self.para_mode.ep_async_mode, self.layer_idx, self.total_layers)
        mask, skip_now = None, None
        if diep.ep_skip_enabled():
            mask = diep.ep_skip_mask_on(x.shape[0] * self.num_experts_per_tok, x.device)
            skip_now = diep.ep_skip_now(self.layer_idx)
        if async_op:
            return self._run_lagged(x, mask, skip_now, caller=caller, y=y).view(*orig_shape)
        mode, cache_in, cache_out = MODE_PLAIN, None, None
        if mask is not None:
            # conditional communication: reference ep_fwd.py:49-66,176-188
            if skip_now:
                mode, cache_in = MODE_SKIP, diep.ep_skip_get(self.layer_idx)
            else:
                mode, cache_out = MODE_PUT, self._cache_buffer(x)
        y = self.run(x, mode, mask, cache_in, cache_out, y=y, caller=caller)
        if mode == MODE_PUT:
            diep.ep_skip_put(self.layer_idx, cache_out)
        elif mode == MODE_SKIP:
            self._spare_cache = cache_in      # consumed (the cache entry is empty now): the next full step refills it
        return y.view(*orig_shape)

    def _cache_buffer(self, x):
        """Where a full step writes the skip cache: the tensor the last skip
        step consumed when it still fits, else a new one.  Everything runs on
        one stream, so the skip step's read is over before the refill starts."""
        spare, self._spare_cache = self._spare_cache, None
        if spare is not None and spare.shape == x.shape and spare.dtype == x.dtype and spare.device == x.device:
            return spare
        return torch.empty_like(x)

    def _check_skip_args(self, x, mode, skip_mask, cache_in, cache_out):
        """The kernels index the mask by slot and the cache by token row of THIS
        call; a mask or cache of another batch would be read out of bounds."""
        n, k = x.shape[0], self.num_experts_per_tok
        if mode != MODE_PLAIN and skip_mask is None:
            raise DiceError("a put or skip step needs the skip mask")
        if skip_mask is not None and (skip_mask.numel() != n * k or skip_mask.device != x.device
                                      or skip_mask.dtype not in (torch.uint8, torch.bool)):
            raise DiceError(f"skip mask: {skip_mask.numel()} entries of {skip_mask.dtype} on {skip_mask.device}, "
                            f"this call needs {n * k} bool / uint8 entries on {x.device}")
        for name, c, wanted in (("cache_in", cache_in, mode == MODE_SKIP), ("cache_out", cache_out, mode == MODE_PUT)):
            if wanted and c is None:
                raise DiceError(f"layer {self.layer_idx}: this step needs {name}")
            if c is not None and (c.shape != x.shape or c.dtype != x.dtype or c.device != x.device):
                raise DiceError(f"layer {self.layer_idx}: {name} is {tuple(c.shape)} {c.dtype} on {c.device}, the "
                                f"layer input {tuple(x.shape)} {x.dtype} on {x.device}: the batch changed since the "
                                "cache was filled; call ep_cache_clear() and run a full step")

    @torch.no_grad()
    def _run_lagged(self, x, mask, skip_now, topk_idx_out=None, topk_weight_out=None, caller=None, y=None):
        """Step-lagged call (reference ep_fwd.py:133-195 with async_op=True):
        this call's routing is booked into the caches, the routed experts run on
        the entry ``diep.lag_roles`` hands back and an older entry is returned.
        The blend with / write of the skip cache follows the EMITTED entry: it
        takes the cache when that entry was dispatched without the skipped
        slots (ep_fwd.py:177-185), else it refills the cache (:186-188)."""
        desc = self._ensure(x)
        n = x.shape[0]
        ws = self._workspace(desc, n, x.device)
        new = self._take_entry(x, bool(skip_now))
        work, emit = diep.lag_roles(self.layer_idx, new)
        for entry in (work, emit):
            if entry.x.shape != x.shape or entry.x.dtype != x.dtype or entry.x.device != x.device:
                raise DiceError(f"layer {self.layer_idx}: a cached step holds {tuple(entry.x.shape)} {entry.x.dtype} "
                                f"activations, this call {tuple(x.shape)} {x.dtype}: clear the caches and force a "
                                "synchronous step when the batch changes")
        work.ensure_rows()
        if emit.rows is None:
            raise DiceError("the cached step to return has never been through the experts")
        mode, cache_in, cache_out = MODE_PLAIN, None, None
        if mask is not None:
            if emit.dropped:
                mode, cache_in = MODE_SKIP, diep.ep_skip_get(self.layer_idx)
                if cache_in is None:
                    raise DiceError(f"layer {self.layer_idx}: a step dispatched without its skipped slots "
                                    "came back but the skip cache is empty")
            else:
                mode, cache_out = MODE_PUT, self._cache_buffer(x)
            if mask.dtype == torch.bool:
                mask = mask.view(torch.uint8)
        self._check_skip_args(x, mode, mask, cache_in, cache_out)
        owner = work.owner if work.owner is not None else self
        experts_of = owner._ensure(x)
        put_d, work_d, emit_d = new.desc(), work.desc(), emit.desc()
        if y is None:
            y = torch.empty_like(x)
        check(load().dice_moe_forward_lagged(
            ctypes.byref(desc), ctypes.byref(experts_of), ptr(x), n, int(bool(skip_now)), ptr(mask),
            ctypes.byref(put_d), None if work is new else ctypes.byref(work_d),
            None if emit is work else ctypes.byref(emit_d), mode, ptr(cache_in), ptr(cache_out),
            int(diep.latest_expert_weights()), None if caller is None else ctypes.byref(caller), ptr(y),
            ptr(topk_idx_out), ptr(topk_weight_out), ptr(ws), ws.numel(), stream_ptr()))
        if mode == MODE_PUT:
            diep.ep_skip_put(self.layer_idx, cache_out)
        elif mode == MODE_SKIP:
            self._spare_cache = cache_in
        if emit is not work and emit is not new and not diep.lag_entry_cached(emit):
            # The returned entry has left both caches: its buffers serve a later call of the
            # block that made it (work queued on the one stream is ordered before any re-use).
            home = emit.owner if emit.owner is not None else self
            if len(home._spare_entries) < 2:
                home._spare_entries.append(emit)
        return y

    def _take_entry(self, x, dropped: bool):
        """A step-lag entry for this call: a retired one of the same shape when
        there is one (its seven buffers are re-used), else a new one."""
        k = self.num_experts_per_tok
        while self._spare_entries:
            e = self._spare_entries.pop()
            if (e.x.shape == x.shape and e.x.dtype == x.dtype and e.x.device == x.device
                    and e.perm.numel() == x.shape[0] * k and e.offsets.numel() == len(self.experts) + 1):
                e.recycle(k, dropped, self)
                return e
        return diep.LagEntry(x, len(self.experts), k, dropped, owner=self)

    @torch.no_grad()
    def run(self, x, mode=MODE_PLAIN, skip_mask=None, cache_in=None, cache_out=None,
            topk_idx_out=None, topk_weight_out=None, y=None, caller=None):
        """One call of ``dice_moe_forward`` on ``x [N, D]`` (of
        ``dice_moe_forward_modulated`` when the caller's prologue / epilogue come
        along: ``x`` is then the residual stream)."""
        desc = self._ensure(x)
        n = x.shape[0]
        self._check_skip_args(x, mode, skip_mask, cache_in, cache_out)
        ws = self._workspace(desc, n, x.device)
        if y is None:
            y = torch.empty_like(x)
        if skip_mask is not None and skip_mask.dtype == torch.bool:
            skip_mask = skip_mask.view(torch.uint8)
        if caller is None:
            check(load().dice_moe_forward(ctypes.byref(desc), ptr(x), n, mode, ptr(skip_mask), ptr(cache_in),
                                          ptr(cache_out), ptr(y), ptr(topk_idx_out), ptr(topk_weight_out),
                                          ptr(ws), ws.numel(), stream_ptr()))
        else:
            check(load().dice_moe_forward_modulated(
                ctypes.byref(desc), ctypes.byref(caller), ptr(x), n, mode, ptr(skip_mask), ptr(cache_in),
                ptr(cache_out), ptr(y), ptr(topk_idx_out), ptr(topk_weight_out), ptr(ws), ws.numel(),
                stream_ptr()))
        return y

    @torch.no_grad()
    def moe_infer(self, x, flat_expert_indices, flat_expert_weights):
        """Routed experts only, from given routing (reference models.py:361-382)."""
        k = self.num_experts_per_tok
        n = x.shape[0]
        if flat_expert_indices.numel() != n * k or flat_expert_weights.numel() != n * k:
            raise DiceError(f"moe_infer: {flat_expert_indices.numel()} indices and {flat_expert_weights.numel()} "
                            f"weights for {n} tokens x {k}")
        idx = flat_expert_indices.reshape(-1).to(torch.int32).contiguous()
        _, offsets, perm, inv_perm = ops.dispatch(idx, len(self.experts))
        rows = self.routed_experts(x.contiguous(), perm, offsets, n * k)
        w = flat_expert_weights.reshape(n, k).float().contiguous()
        return ops.combine(rows, w, n, k, inv_perm=inv_perm)
