"""Sliding-window attention, public entry points (single-GPU path).

Same names, positional order and argument meaning as the upstream package
(``ring_swa/sliding_window/nonvarlen.py:341-408`` and
``ring_swa/sliding_window/varlen.py:362-441``).  With ``cp_group=None`` the call
runs the HIP band-attention kernels directly; with a ``cp_group`` it goes through
``ring_swa/ring.py`` (one process per GPU, chunks exchanged over ``torch.distributed``).
"""
from __future__ import annotations

from typing import Optional

import torch

from .ops.band_attn import attn_bwd, attn_fwd


class BandAttnFunc(torch.autograd.Function):
    """Causal band attention (optionally with sink keys) as one autograd node.

    Forward = one ``attn_fwd`` launch; backward = one ``attn_bwd`` call fed the
    saved ``(out, lse)``.
    """

    @staticmethod
    def forward(ctx, q, k, v, window_size, softmax_scale, cu_seqlens, num_sink):
        if softmax_scale is None:
            softmax_scale = q.shape[-1] ** (-0.5)
        out, lse = attn_fwd(q, k, v, softmax_scale, (window_size, 0), True, cu_seqlens,
                            cu_seqlens, num_sink=num_sink)
        ctx.save_for_backward(q, k, v, out, lse)
        ctx.cu_seqlens = cu_seqlens
        ctx.meta = (window_size, softmax_scale, num_sink)
        return out

    @staticmethod
    def backward(ctx, do):
        q, k, v, out, lse = ctx.saved_tensors
        window_size, softmax_scale, num_sink = ctx.meta
        if do.stride(-1) != 1:
            do = do.contiguous()
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        attn_bwd(q, k, v, out, lse, do, dq, dk, dv, softmax_scale, (window_size, 0), True,
                 ctx.cu_seqlens, ctx.cu_seqlens, num_sink=num_sink)
        return dq, dk, dv, None, None, None, None


def _ring_ranks(cp_group, cp_size, cp_local_rank, cp_prev_global_rank, cp_next_global_rank):
    """The rank arguments of a call with ``cp_group``: ``cp_size`` and ``cp_local_rank`` default
    to the group's own, and the neighbours' global ranks, if given, must be the ones the
    group's rank map yields (``README.md:63-64`` of the upstream package obtains them from it)."""
    import torch.distributed as dist

    from .ops.p2p import get_group_local_to_global_rank_map

    if cp_size is None:
        cp_size = dist.get_world_size(cp_group)
    if cp_local_rank is None:
        cp_local_rank = dist.get_rank(cp_group)
    gmap = get_group_local_to_global_rank_map(cp_group)
    for given, other in ((cp_prev_global_rank, (cp_local_rank - 1) % cp_size),
                         (cp_next_global_rank, (cp_local_rank + 1) % cp_size)):
        assert given is None or given == gmap[other], (
            f"neighbour rank {given} is not the group's rank {other} (global {gmap[other]})"
        )
    return int(cp_size), int(cp_local_rank)


def _check_dense(q, k, v):
    assert q.dim() == 4 and k.dim() == 4 and v.dim() == 4, "expected [batch, seq, heads, dim]"
    assert q.shape[1] == k.shape[1] == v.shape[1], "Sequence length must be the same"
    assert q.shape[2] % k.shape[2] == 0, (
        "Number of query heads must be divisible by number of key/value heads"
    )


def _check_packed(q, k, v, cu_seqlens, cp_size):
    assert q.dim() == 3 and k.dim() == 3 and v.dim() == 3, "expected [tokens, heads, dim]"
    assert q.shape[0] == k.shape[0] == v.shape[0], "Sequence length must be the same"
    assert q.shape[1] % k.shape[1] == 0, (
        "Number of query heads must be divisible by number of key/value heads"
    )
    assert cu_seqlens.dtype == torch.int32 and cu_seqlens.dim() == 1, "cu_seqlens must be int32 [B+1]"
    # Upstream evaluates `cu_seqlens[-1] // cp_size` (a device read) before looking at
    # cp_group, and fails with a TypeError when cp_size is left at None; here a missing
    # cp_size means 1 on the single-GPU path and the check is done without touching the
    # device: the packed tensors must hold cu_seqlens[-1] rows, which the kernel bounds
    # by q.shape[0] anyway.
    assert cp_size in (None, 1), "cp_size > 1 needs cp_group"


def ring_sliding_window_attn(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    window_size: int,
    cp_group=None,
    cp_size: Optional[int] = None,
    cp_local_rank: Optional[int] = None,
    cp_prev_global_rank: Optional[int] = None,
    cp_next_global_rank: Optional[int] = None,
    softmax_scale: Optional[float] = None,
) -> torch.Tensor:
    """Causal sliding-window attention, ``[batch, seq, heads, dim]`` tensors.

    Each query attends ``window_size + 1`` keys including itself, as flash-attn's
    ``window_size=(w, 0), causal=True`` (``ring_swa/sliding_window/nonvarlen.py:376-386``).
    Returns the attention output, same shape and dtype as ``q``.
    """
    _check_dense(q, k, v)
    if cp_group is not None:
        from .ring import ring_attn

        cp_size, cp_local_rank = _ring_ranks(cp_group, cp_size, cp_local_rank,
                                             cp_prev_global_rank, cp_next_global_rank)
        return ring_attn(q, k, v, window_size, cp_group, cp_size, cp_local_rank, softmax_scale)
    return BandAttnFunc.apply(q, k, v, int(window_size), softmax_scale, None, 0)


def ring_sliding_window_attn_varlen(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    window_size: int,
    cu_seqlens: torch.Tensor,
    cp_group=None,
    cp_size: Optional[int] = None,
    cp_local_rank: Optional[int] = None,
    cp_prev_global_rank: Optional[int] = None,
    cp_next_global_rank: Optional[int] = None,
    softmax_scale: Optional[float] = None,
) -> torch.Tensor:
    """Packed variant: ``[tokens, heads, dim]`` tensors, ``cu_seqlens`` int32 ``[B+1]``.

    ``ring_swa/sliding_window/varlen.py:401-417``.  No host synchronisation: the
    longest sequence length is never read back.
    """
    if cp_group is not None:
        from .ring import ring_attn

        _check_packed(q, k, v, cu_seqlens, 1)
        cp_size, cp_local_rank = _ring_ranks(cp_group, cp_size, cp_local_rank,
                                             cp_prev_global_rank, cp_next_global_rank)
        return ring_attn(q, k, v, window_size, cp_group, cp_size, cp_local_rank, softmax_scale,
                         cu_seqlens)
    _check_packed(q, k, v, cu_seqlens, cp_size)
    return BandAttnFunc.apply(q, k, v, int(window_size), softmax_scale, cu_seqlens.contiguous(), 0)
