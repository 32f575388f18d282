"""Kernel-level operators of the single-GPU path (HIP, gfx950)."""
from .lse_merge import merge_attn_out

__all__ = ["merge_attn_out"]
