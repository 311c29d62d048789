"""ctypes binding of ``libdice_moe.so`` (the C ABI declared in include/dice_moe.h).

The library is the product path.  There is no CPU or eager-torch fallback: if
the shared object is missing or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, Structure, c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_void_p
from typing import Optional

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libdice_moe.so")

DICE_F32, DICE_BF16, DICE_F16, DICE_FP8_E4M3 = 0, 1, 2, 3
DICE_ACT_SWIGLU, DICE_ACT_GELU_TANH = 0, 1
MODE_PLAIN, MODE_PUT, MODE_SKIP = 0, 1, 2

_DTYPES = {
    torch.float32: DICE_F32,
    torch.bfloat16: DICE_BF16,
    torch.float16: DICE_F16,
    torch.float8_e4m3fn: DICE_FP8_E4M3,
}

EXPORTS = [
    "dice_abi_version",
    "dice_last_error",
    "dice_gate_topk",
    "dice_dispatch_workspace_bytes",
    "dice_dispatch",
    "dice_dispatch_static_scratch_bytes",
    "dice_dispatch_static",
    "dice_gather_rows",
    "dice_grouped_mlp",
    "dice_grouped_mlp_stage",
    "dice_set_gemm_config",
    "dice_debug_persist_turns",
    "dice_profile_enable",
    "dice_profile_stage_count",
    "dice_profile_stage_name",
    "dice_profile_read",
    "dice_combine",
    "dice_quantize_fp8_rowwise",
    "dice_quantize_fp8_act",
    "dice_grouped_mlp_a8",
    "dice_moe_workspace_bytes",
    "dice_moe_forward",
    "dice_moe_forward_lagged",
    "dice_ln_modulate",
    "dice_combine_residual",
    "dice_moe_forward_modulated",
]


class DiceError(RuntimeError):
    pass


class MoeLayerDesc(Structure):
    """Mirror of ``dice_moe_layer_t``."""

    _fields_ = [
        ("hidden", c_int32), ("inter", c_int32), ("n_experts", c_int32), ("top_k", c_int32),
        ("act_dtype", c_int32), ("w_dtype", c_int32), ("act_variant", c_int32),
        ("norm_topk_prob", c_int32), ("gate_w_dtype", c_int32), ("shared_inter", c_int32),
        ("gate_w", c_void_p), ("gate_bias", c_void_p),
        ("w1", c_void_p), ("w2", c_void_p),
        ("b1", c_void_p), ("b2", c_void_p), ("w1_scale", c_void_p), ("w2_scale", c_void_p),
        ("shared_w1", c_void_p), ("shared_w2", c_void_p),
        ("shared_b1", c_void_p), ("shared_b2", c_void_p),
        ("act_quant", c_int32), ("batch_invariant", c_int32),
    ]


class LagEntryDesc(Structure):
    """Mirror of ``dice_moe_lag_entry_t``."""

    _fields_ = [
        ("x", c_void_p), ("offsets", c_void_p), ("perm", c_void_p), ("inv_perm", c_void_p),
        ("topk_weight", c_void_p), ("rows", c_void_p), ("max_rows", c_int64),
    ]


class CallerDesc(Structure):
    """Mirror of ``dice_moe_caller_t``."""

    _fields_ = [("shift", c_void_p), ("scale", c_void_p), ("gate", c_void_p),
                ("tokens_per_sample", c_int64), ("ln_eps", c_float)]


_lib: Optional[ctypes.CDLL] = None


def load() -> ctypes.CDLL:
    """Loads the shared library once and declares every prototype."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise DiceError(
            f"{LIB_PATH} is missing: build it with `python -m dice_amd.build` "
            "(there is no fallback path)")
    lib = ctypes.CDLL(LIB_PATH)
    lib.dice_abi_version.restype = c_int
    lib.dice_last_error.restype = c_char_p
    lib.dice_gate_topk.restype = c_int
    lib.dice_gate_topk.argtypes = [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int64, c_int, c_int,
                                   c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
    lib.dice_dispatch_workspace_bytes.restype = c_size_t
    lib.dice_dispatch_workspace_bytes.argtypes = [c_int64, c_int]
    lib.dice_dispatch.restype = c_int
    lib.dice_dispatch.argtypes = [c_void_p, c_void_p, c_int64, c_int, c_void_p, c_void_p, c_void_p,
                                  c_void_p, c_void_p, c_size_t, c_void_p]
    lib.dice_dispatch_static_scratch_bytes.restype = c_size_t
    lib.dice_dispatch_static_scratch_bytes.argtypes = []
    lib.dice_dispatch_static.restype = c_int
    lib.dice_dispatch_static.argtypes = [c_void_p, c_void_p, c_int64, c_int, c_void_p, c_void_p, c_void_p,
                                         c_void_p, c_void_p]
    lib.dice_gather_rows.restype = c_int
    lib.dice_gather_rows.argtypes = [c_void_p, c_int, c_void_p, c_int, c_int64, c_int, c_void_p, c_void_p]
    lib.dice_grouped_mlp.restype = c_int
    lib.dice_grouped_mlp.argtypes = [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int64, c_int,
                                     c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                     c_int, c_int, c_void_p, c_void_p, c_int, c_void_p]
    lib.dice_grouped_mlp_stage.restype = c_int
    lib.dice_grouped_mlp_stage.argtypes = [c_int] + lib.dice_grouped_mlp.argtypes
    lib.dice_combine.restype = c_int
    lib.dice_combine.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                 c_void_p, c_int, c_int64, c_int, c_int, c_void_p]
    lib.dice_quantize_fp8_rowwise.restype = c_int
    lib.dice_quantize_fp8_rowwise.argtypes = [c_void_p, c_int, c_int64, c_int64, c_void_p, c_void_p, c_void_p]
    lib.dice_quantize_fp8_act.restype = c_int
    lib.dice_quantize_fp8_act.argtypes = [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int64, c_int, c_void_p,
                                          c_void_p, c_void_p]
    lib.dice_grouped_mlp_a8.restype = c_int
    lib.dice_grouped_mlp_a8.argtypes = [c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int64, c_int,
                                        c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                        c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
    lib.dice_moe_workspace_bytes.restype = c_size_t
    lib.dice_moe_workspace_bytes.argtypes = [POINTER(MoeLayerDesc), c_int64]
    lib.dice_moe_forward.restype = c_int
    lib.dice_moe_forward.argtypes = [POINTER(MoeLayerDesc), c_void_p, c_int64, c_int, c_void_p, c_void_p,
                                     c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]
    lib.dice_moe_forward_lagged.restype = c_int
    lib.dice_moe_forward_lagged.argtypes = [POINTER(MoeLayerDesc), POINTER(MoeLayerDesc), c_void_p, c_int64,
                                            c_int, c_void_p, POINTER(LagEntryDesc), POINTER(LagEntryDesc),
                                            POINTER(LagEntryDesc), c_int, c_void_p, c_void_p, c_int,
                                            POINTER(CallerDesc), c_void_p, c_void_p, c_void_p, c_void_p,
                                            c_size_t, c_void_p]
    lib.dice_ln_modulate.restype = c_int
    lib.dice_ln_modulate.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int, c_int64,
                                     c_float, c_void_p]
    lib.dice_combine_residual.restype = c_int
    lib.dice_combine_residual.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                          c_void_p, c_void_p, c_int64, c_void_p, c_int, c_int64, c_int, c_int,
                                          c_void_p]
    lib.dice_moe_forward_modulated.restype = c_int
    lib.dice_moe_forward_modulated.argtypes = [POINTER(MoeLayerDesc), POINTER(CallerDesc), c_void_p, c_int64,
                                               c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                               c_void_p, c_void_p, c_size_t, c_void_p]
    lib.dice_profile_enable.restype = c_int
    lib.dice_profile_enable.argtypes = [c_int]
    lib.dice_profile_stage_count.restype = c_int
    lib.dice_profile_stage_name.restype = c_char_p
    lib.dice_profile_stage_name.argtypes = [c_int]
    lib.dice_profile_read.restype = c_int
    lib.dice_profile_read.argtypes = [POINTER(c_float), c_int]
    lib.dice_set_gemm_config.restype = c_int
    lib.dice_set_gemm_config.argtypes = [c_int, c_int]
    lib.dice_debug_persist_turns.restype = c_int
    lib.dice_debug_persist_turns.argtypes = [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                             c_void_p, c_void_p]
    if lib.dice_abi_version() != 2:
        raise DiceError(f"ABI version {lib.dice_abi_version()} != 2")
    _lib = lib
    return lib


def check(rc: int) -> None:
    if rc != 0:
        msg = load().dice_last_error()
        raise DiceError(f"libdice_moe error {rc}: {msg.decode() if msg else ''}")


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _DTYPES[dt]
    except KeyError:
        raise DiceError(f"unsupported dtype {dt}") from None


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    """Device address of a contiguous CUDA(HIP) tensor, or NULL."""
    if t is None:
        return None
    if not t.is_cuda:
        raise DiceError("libdice_moe needs device tensors; this build has no CPU path")
    if not t.is_contiguous():
        raise DiceError("libdice_moe needs contiguous tensors")
    return t.data_ptr()


def stream_ptr() -> int:
    return torch.cuda.current_stream().cuda_stream
