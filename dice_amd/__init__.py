"""MI355X-native DiT-MoE sparse expert layer (HIP kernels behind a C ABI)."""
from . import checkpoint, diep, ep_fwd, graphs, lib, ops  # noqa: F401
from .lib import DiceError  # noqa: F401
from .moe import GeluMLP, MoEGate, MoeMLP, ParaMode, SparseMoeBlock  # noqa: F401

__all__ = ["SparseMoeBlock", "MoEGate", "MoeMLP", "GeluMLP", "ParaMode", "DiceError", "diep", "ep_fwd", "ops", "lib", "checkpoint", "graphs"]
