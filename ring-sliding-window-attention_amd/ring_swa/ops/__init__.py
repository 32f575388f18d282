"""Kernel-level operators of the single-GPU path (HIP, gfx950)."""
from .band_attn import (
    attn_bwd,
    attn_fwd,
    wrapped_flash_attn_bwd,
    wrapped_flash_attn_bwd_varlen,
    wrapped_flash_attn_fwd,
    wrapped_flash_attn_fwd_varlen,
)
from .lse_merge import merge_attn_out

__all__ = [
    "attn_fwd",
    "attn_bwd",
    "wrapped_flash_attn_fwd",
    "wrapped_flash_attn_fwd_varlen",
    "wrapped_flash_attn_bwd",
    "wrapped_flash_attn_bwd_varlen",
    "merge_attn_out",
]
