"""Sliding-window attention, public entry points (single-GPU path).

Same names, positional order and argument meaning as the upstream package
(``ring_swa/sliding_window/nonvarlen.py:341-408`` and
``ring_swa/sliding_window/varlen.py:362-441``).  With ``cp_group=None`` the call
runs the HIP band-attention kernels directly; the multi-GPU ring
(``cp_group`` given) is not part of this build and raises.
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


def _reject_ring(cp_group):
    if cp_group is not None:
        raise NotImplementedError(
            "this build covers the single-GPU path (cp_group=None) and one rank's share of the "
            "ring (ring_swa.rank_share); the multi-GPU ring itself is not implemented"
        )


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
    assert cp_size in (None, 1), "cp_size > 1 needs cp_group (not part of this build)"


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
    _reject_ring(cp_group)
    _check_dense(q, k, v)
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
    _reject_ring(cp_group)
    _check_packed(q, k, v, cu_seqlens, cp_size)
    return BandAttnFunc.apply(q, k, v, int(window_size), softmax_scale, cu_seqlens.contiguous(), 0)
