"""Streaming-LLM attention (attention sinks + sliding window), public entry points.

Same names, positional order and argument meaning as the upstream package
(``ring_swa/streaming_llm/nonvarlen.py:400-468``,
``ring_swa/streaming_llm/varlen.py:476-552``); with ``cp_group=None`` upstream
runs ``ring_swa/streaming_llm/naive.py``.  Each query attends the first
``num_sink_tokens`` tokens of its own sequence plus the causal window of
``window_size + 1`` keys.

Two execution strategies, selected by the keyword-only ``impl``:

``"fused"`` (default)
    one kernel launch per direction: the sink keys are extra key tiles of the
    band kernel, no partials, no merge.
``"split"``
    the structure of ``ring_swa/streaming_llm/naive.py``: a window partial and a
    sink partial combined by the LSE merge kernel; backward runs one kernel call
    per partial with the merged ``(o, lse)``.  The sink partial only covers the
    sink keys that lie *outside* the query's window, so no key is counted twice
    and any ``num_sink_tokens`` works.

Upstream supports exactly one sink token and, in the packed forward, takes the
sink of every sequence from the first token of the pack
(``ring_swa/streaming_llm/naive.py:116-117``, valid when all sequences start
with the same token).  Here every sequence uses its own first tokens; under
upstream's precondition the results coincide.
"""
from __future__ import annotations

from typing import Optional

import torch

from .ops.band_attn import attn_bwd, attn_fwd
from .ops.lse_merge import merge_attn_out
from .sliding_window import BandAttnFunc, _check_dense, _check_packed, _ring_ranks


class SinkWindowSplitFunc(torch.autograd.Function):
    """Window partial + out-of-window sink partial, merged by LSE (dense tensors)."""

    @staticmethod
    def forward(ctx, q, k, v, window_size, softmax_scale, num_sink):
        if softmax_scale is None:
            softmax_scale = q.shape[-1] ** (-0.5)
        n = min(num_sink, k.shape[1])
        o, lse = attn_fwd(q, k, v, softmax_scale, (window_size, 0), True)
        # keys j < n with j <= i - window_size - 1: diagonal moved w + 1 to the left
        o_s, lse_s = attn_fwd(q, k[:, :n], v[:, :n], softmax_scale, (-1, 0), False,
                              mask_shift=-(window_size + 1))
        merge_attn_out(o, lse, o_s, lse_s)
        ctx.save_for_backward(q, k, v, o, lse)
        ctx.meta = (window_size, softmax_scale, n)
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, lse = ctx.saved_tensors
        window_size, softmax_scale, n = ctx.meta
        if do.stride(-1) != 1:
            do = do.contiguous()
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        attn_bwd(q, k, v, o, lse, do, dq, dk, dv, softmax_scale, (window_size, 0), True)
        dq_s = torch.empty_like(q)
        dk_s, dv_s = torch.empty_like(k[:, :n]), torch.empty_like(v[:, :n])
        attn_bwd(q, k[:, :n], v[:, :n], o, lse, do, dq_s, dk_s, dv_s, softmax_scale, (-1, 0),
                 False, mask_shift=-(window_size + 1))
        dq.add_(dq_s)
        dk[:, :n].add_(dk_s)
        dv[:, :n].add_(dv_s)
        return dq, dk, dv, None, None, None


class SinkWindowSplitVarlenFunc(torch.autograd.Function):
    """Packed twin of :class:`SinkWindowSplitFunc`; per-sequence sink keys are gathered
    into a small packed tensor (``num_sink`` rows per sequence) without reading
    ``cu_seqlens`` back to the host."""

    @staticmethod
    def forward(ctx, q, k, v, window_size, cu_seqlens, softmax_scale, num_sink):
        if softmax_scale is None:
            softmax_scale = q.shape[-1] ** (-0.5)
        n = int(num_sink)
        nseq = cu_seqlens.numel() - 1
        starts = cu_seqlens[:-1].long()
        last = (cu_seqlens[1:].long() - 1).clamp_min(0)
        # rows past the end of a short sequence repeat its last token; the mask never shows them
        idx = torch.minimum(starts[:, None] + torch.arange(n, device=q.device)[None, :],
                            last[:, None]).reshape(-1)
        cu_sink = torch.arange(0, (nseq + 1) * n, n, device=q.device, dtype=torch.int32)
        k_s, v_s = k[idx], v[idx]
        o, lse = attn_fwd(q, k, v, softmax_scale, (window_size, 0), True, cu_seqlens, cu_seqlens)
        o_s, lse_s = attn_fwd(q, k_s, v_s, softmax_scale, (-1, 0), False, cu_seqlens, cu_sink,
                              mask_shift=-(window_size + 1))
        merge_attn_out(o.unsqueeze(0), lse.unsqueeze(0), o_s.unsqueeze(0), lse_s.unsqueeze(0))
        ctx.save_for_backward(q, k, v, o, lse, k_s, v_s, cu_seqlens, cu_sink, idx)
        ctx.meta = (window_size, softmax_scale)
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, lse, k_s, v_s, cu_seqlens, cu_sink, idx = ctx.saved_tensors
        window_size, softmax_scale = ctx.meta
        if do.stride(-1) != 1:
            do = do.contiguous()
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        attn_bwd(q, k, v, o, lse, do, dq, dk, dv, softmax_scale, (window_size, 0), True,
                 cu_seqlens, cu_seqlens)
        dq_s, dk_s, dv_s = torch.empty_like(q), torch.empty_like(k_s), torch.empty_like(v_s)
        attn_bwd(q, k_s, v_s, o, lse, do, dq_s, dk_s, dv_s, softmax_scale, (-1, 0), False,
                 cu_seqlens, cu_sink, mask_shift=-(window_size + 1))
        dq.add_(dq_s)
        dk.index_add_(0, idx, dk_s)  # repeated rows carry zero gradient
        dv.index_add_(0, idx, dv_s)
        return dq, dk, dv, None, None, None, None


def _impl(impl: str) -> bool:
    if impl not in ("fused", "split"):
        raise ValueError(f"impl must be 'fused' or 'split', got {impl!r}")
    return impl == "fused"


def ring_streaming_llm_attn(
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
    *,
    num_sink_tokens: int = 1,
    impl: str = "fused",
) -> torch.Tensor:
    """Sink + sliding-window attention on ``[batch, seq, heads, dim]`` tensors.  With a
    ``cp_group`` the tensors are this rank's chunk of the sequence (``ring_slm.py``; ``impl``
    plays no role there)."""
    _check_dense(q, k, v)
    assert num_sink_tokens >= 0
    _impl(impl)
    if cp_group is not None:
        from .ring_slm import ring_slm_attn

        cp_size, cp_local_rank = _ring_ranks(cp_group, cp_size, cp_local_rank,
                                             cp_prev_global_rank, cp_next_global_rank)
        return ring_slm_attn(q, k, v, window_size, cp_group, cp_size, cp_local_rank,
                             softmax_scale, num_sink_tokens=num_sink_tokens)
    if _impl(impl) or num_sink_tokens == 0:
        return BandAttnFunc.apply(q, k, v, int(window_size), softmax_scale, None,
                                  int(num_sink_tokens))
    return SinkWindowSplitFunc.apply(q, k, v, int(window_size), softmax_scale,
                                     int(num_sink_tokens))


def ring_streaming_llm_attn_varlen(
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
    *,
    num_sink_tokens: int = 1,
    impl: str = "fused",
) -> torch.Tensor:
    """Packed variant: ``[tokens, heads, dim]`` tensors, ``cu_seqlens`` int32 ``[B+1]`` (with a
    ``cp_group``: of the whole pack, the tensors being this rank's chunk of it)."""
    assert num_sink_tokens >= 0
    _impl(impl)
    if cp_group is not None:
        from .ring_slm import ring_slm_attn

        _check_packed(q, k, v, cu_seqlens, 1)
        cp_size, cp_local_rank = _ring_ranks(cp_group, cp_size, cp_local_rank,
                                             cp_prev_global_rank, cp_next_global_rank)
        return ring_slm_attn(q, k, v, window_size, cp_group, cp_size, cp_local_rank,
                             softmax_scale, cu_seqlens, num_sink_tokens=num_sink_tokens)
    _check_packed(q, k, v, cu_seqlens, cp_size)
    cu = cu_seqlens.contiguous()
    if _impl(impl) or num_sink_tokens == 0:
        return BandAttnFunc.apply(q, k, v, int(window_size), softmax_scale, cu,
                                  int(num_sink_tokens))
    return SinkWindowSplitVarlenFunc.apply(q, k, v, int(window_size), cu, softmax_scale,
                                           int(num_sink_tokens))
