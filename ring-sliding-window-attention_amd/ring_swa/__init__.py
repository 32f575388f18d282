"""MI355X-native single-GPU attention path of ring_swa.

The four public functions keep upstream's names and signatures
(``ring_swa/__init__.py:1-9``); ``ring_rank_share_attn[_varlen]`` expose one
context-parallel rank's share of the ring on a single GPU.
"""
from .rank_share import ring_rank_share_attn, ring_rank_share_attn_varlen
from .sliding_window import ring_sliding_window_attn, ring_sliding_window_attn_varlen
from .streaming_llm import ring_streaming_llm_attn, ring_streaming_llm_attn_varlen

__all__ = [
    "ring_sliding_window_attn",
    "ring_sliding_window_attn_varlen",
    "ring_streaming_llm_attn",
    "ring_streaming_llm_attn_varlen",
    "ring_rank_share_attn",
    "ring_rank_share_attn_varlen",
]
