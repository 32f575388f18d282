"""Kernel-level operators of the attention path (HIP, gfx950) and the operators of the ring
loops built on them; same names as the upstream package exports from ``ring_swa.ops``."""
from .accum import (
    flash_attn_bwd_func,
    flash_attn_fwd_func,
    flash_attn_varlen_bwd_func,
    flash_attn_varlen_fwd_func,
)
from .band_attn import (
    attn_bwd,
    attn_fwd,
    wrapped_flash_attn_bwd,
    wrapped_flash_attn_bwd_varlen,
    wrapped_flash_attn_fwd,
    wrapped_flash_attn_fwd_varlen,
)
from .lse_merge import merge_attn_out
from .p2p import (
    broadcast_tensor_to_group,
    exchange_and_sum_tensors,
    get_group_local_to_global_rank_map,
    reduce_sum_tesnsor_to_rank,
    ring_attn_p2p_communicate,
)

__all__ = [
    "attn_fwd",
    "attn_bwd",
    "wrapped_flash_attn_fwd",
    "wrapped_flash_attn_fwd_varlen",
    "wrapped_flash_attn_bwd",
    "wrapped_flash_attn_bwd_varlen",
    "flash_attn_fwd_func",
    "flash_attn_bwd_func",
    "flash_attn_varlen_fwd_func",
    "flash_attn_varlen_bwd_func",
    "merge_attn_out",
    "ring_attn_p2p_communicate",
    "broadcast_tensor_to_group",
    "reduce_sum_tesnsor_to_rank",
    "exchange_and_sum_tensors",
    "get_group_local_to_global_rank_map",
]
