"""Sliding-window attention over a context-parallel group (``cp_group`` given): every rank
holds one contiguous chunk of the sequence, attends its own chunk and the trailing keys of
the chunks before it, and hands the gradients of those keys back to their owners.

Same mathematics and block geometry as the upstream ring
(``ring_swa/sliding_window/nonvarlen.py:17-338``, ``varlen.py:19-359``; the per-rank block
plan is ``rank_share.plan_nonvarlen`` / ``plan_varlen``), different data movement.  Upstream
relays whole KV chunks from neighbour to neighbour, one hop per step, and lets fp32 dKV
buffers travel the ring backwards.  Here every rank

* sends each later rank that needs it exactly the key range that rank's block reads (the
  last ``min(w - (i - 1) S, S)`` tokens for the hop-``i`` corner block, the whole chunk for
  full blocks), straight to that rank -- on an MI355X node every pair of GPUs has its own
  xGMI link, so the fetches of several predecessors run side by side instead of one per hop;
* posts all of a phase's sends and receives as one batch, runs its own-chunk block while they
  are in flight, then the blocks on the received ranges;
* in the backward sends the 16-bit dKV of every received range back to its owner, which adds
  the contributions to its own in fp32 in hop order (the sums upstream forms along the ring).

Every plan is computed from ``(seq_len, window, cp_size)`` -- and the global ``cu_seqlens`` of
a pack -- which all ranks know, so a sender needs no message to learn what a receiver wants.

The compute is expressed in the four block operators of ``ops/accum.py`` with upstream's
accumulator types (fp32 output, fp64 LSE).  ``kernels`` selects the primitives under them:
the HIP library by default; the CPU test tier passes stand-ins and runs this file over gloo.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch

from .ops.accum import (flash_attn_bwd_func, flash_attn_fwd_func, flash_attn_varlen_bwd_func,
                        flash_attn_varlen_fwd_func)
from .ops.p2p import exchange, get_group_local_to_global_rank_map
from .rank_share import Step, plan_nonvarlen, plan_varlen, ring_comm_times


def _steps_of(rank: int, seq_len: int, window_size: int, cp_size: int,
              cu_host: Optional[Sequence[int]]) -> Tuple[Optional[List[int]], List[Step]]:
    if cu_host is None:
        return None, plan_nonvarlen(seq_len, window_size, cp_size, rank)
    return plan_varlen(cu_host, seq_len, window_size, cp_size, rank)


def _incoming(rank: int, seq_len: int, window_size: int, cp_size: int, cu_host):
    """``(hop, later rank, key slice of this rank's chunk)`` for every later rank whose plan
    has a block on this rank's keys."""
    out = []
    for j in range(1, ring_comm_times(window_size, seq_len, cp_size) + 1):
        other = rank + j
        if other >= cp_size:
            break
        for (i, _, ks, _, _) in _steps_of(other, seq_len, window_size, cp_size, cu_host)[1]:
            if i == j:
                out.append((j, other, ks))
    return out


def band_forward(q, kv, window_size, cp_group, cp_size, rank, softmax_scale, kernels, cu_host):
    """Forward of the band blocks of one rank on ``[batch, seq, heads, dim]`` chunks (batch 1
    around a packed chunk): returns the accumulators of
    ``ring_swa/sliding_window/nonvarlen.py:53-59`` -- fp32 output, fp64 LSE -- before their
    final cast, the device ``cu_seqlens`` of the own-chunk block (packed), the block plan and
    the received key ranges by hop."""
    b, s, hq, d = q.shape
    local_cu, steps = _steps_of(rank, s, window_size, cp_size, cu_host)
    cu_dev = None
    if cu_host is not None:
        cu_dev = torch.tensor(local_cu, dtype=torch.int32, device=q.device)
    gmap = get_group_local_to_global_rank_map(cp_group)

    # what this rank reads of earlier chunks / what later ranks read of this one
    got = {}
    recvs = []
    for (i, _, ks, _, _) in steps:
        if i > 0:
            got[i] = kv.new_empty((2, b, ks.stop - ks.start, kv.shape[3], d))
            recvs.append((got[i], gmap[rank - i]))
    sends = [(kv[:, :, ks].contiguous(), gmap[other])
             for (_, other, ks) in _incoming(rank, s, window_size, cp_size, cu_host)]
    reqs = exchange(sends, recvs, cp_group)

    out = torch.zeros_like(q, dtype=torch.float32)
    lse = torch.full((b, hq, s), float("-inf"), dtype=torch.float64, device=q.device)
    (_, _, _, window0, causal0) = steps[0]
    if cu_host is not None:
        flash_attn_varlen_fwd_func(q, kv, softmax_scale, window0, cu_dev, cu_dev, None, None,
                                   causal0, out, lse, kernels=kernels)
    else:
        flash_attn_fwd_func(q, kv, softmax_scale, window0, causal0, out, lse, kernels=kernels)
    for req in reqs:
        req.wait()
    for (i, qs, _, window, causal) in steps[1:]:
        flash_attn_fwd_func(q[:, qs], got[i], softmax_scale, window, causal, out[:, qs],
                            lse[:, :, qs], kernels=kernels)
    return out, lse, cu_dev, steps, got


def band_backward(q, kv, out, lse, do, got_list, window_size, cp_group, cp_size, rank,
                  softmax_scale, kernels, cu_host, steps, cu_dev):
    """Backward of the same blocks from the final ``(out, lse)``: fp32 ``dq`` and ``dkv`` of this
    rank's chunk, the contributions of later ranks included."""
    s = q.shape[1]
    gmap = get_group_local_to_global_rank_map(cp_group)
    dq = torch.zeros_like(q, dtype=torch.float32)
    dkv = torch.zeros_like(kv, dtype=torch.float32)

    # blocks on received key ranges first: their dKV goes back to the owners while the
    # own-chunk block runs
    sends = []
    for (i, qs, _, window, causal), kv_i in zip(steps[1:], got_list):
        dq_i = torch.empty_like(q[:, qs])
        dkv_i = torch.empty_like(kv_i)
        flash_attn_bwd_func(q[:, qs], kv_i, out[:, qs], lse[:, :, qs], do[:, qs], dq_i, dkv_i,
                            softmax_scale, window, causal, kernels=kernels)
        dq[:, qs] += dq_i
        sends.append((dkv_i, gmap[rank - i]))
    incoming = _incoming(rank, s, window_size, cp_size, cu_host)
    back = [kv.new_empty((2, kv.shape[1], ks.stop - ks.start, kv.shape[3], kv.shape[4]))
            for (_, _, ks) in incoming]
    recvs = [(buf, gmap[other]) for buf, (_, other, _) in zip(back, incoming)]
    reqs = exchange(sends, recvs, cp_group)

    (_, _, _, window0, causal0) = steps[0]
    dq_0, dkv_0 = torch.empty_like(q), torch.empty_like(kv)
    if cu_host is not None:
        flash_attn_varlen_bwd_func(q, kv, out, lse, do, dq_0, dkv_0, cu_dev, cu_dev, None, None,
                                   softmax_scale, window0, causal0, kernels=kernels)
    else:
        flash_attn_bwd_func(q, kv, out, lse, do, dq_0, dkv_0, softmax_scale, window0, causal0,
                            kernels=kernels)
    dq += dq_0
    dkv += dkv_0
    for req in reqs:
        req.wait()
    for buf, (_, _, ks) in zip(back, incoming):  # hop order: a fixed order of the fp32 sums
        dkv[:, :, ks] += buf
    return dq, dkv


class RingSlidingWindowFunc(torch.autograd.Function):
    """Dense ``[batch, seq, heads, dim]`` chunks, or packed ``[tokens, heads, dim]`` chunks
    when ``cu_host`` (the cumulative lengths of the WHOLE pack, a host list) is given."""

    @staticmethod
    def forward(ctx, q, k, v, window_size, cp_group, cp_size, rank, softmax_scale, kernels,
                cu_host):
        packed = cu_host is not None
        if packed:
            q, k, v = q.unsqueeze(0), k.unsqueeze(0), v.unsqueeze(0)
        if softmax_scale is None:
            softmax_scale = q.shape[-1] ** (-0.5)
        kv = torch.stack([k, v], dim=0)
        out, lse, cu_dev, steps, got = band_forward(q, kv, window_size, cp_group, cp_size, rank,
                                                    softmax_scale, kernels, cu_host)
        out = out.to(q.dtype)
        lse = lse.to(torch.float32)
        ctx.save_for_backward(q, kv, out, lse, *(got[i] for (i, *_rest) in steps[1:]))
        ctx.cu_dev = cu_dev
        ctx.meta = (window_size, cp_group, cp_size, rank, softmax_scale, kernels, cu_host, steps)
        return out.squeeze(0) if packed else out

    @staticmethod
    def backward(ctx, do):
        q, kv, out, lse, *got_list = ctx.saved_tensors
        window_size, cp_group, cp_size, rank, softmax_scale, kernels, cu_host, steps = ctx.meta
        packed = cu_host is not None
        if packed:
            do = do.unsqueeze(0)
        if do.stride(-1) != 1:
            do = do.contiguous()
        dq, dkv = band_backward(q, kv, out, lse, do, got_list, window_size, cp_group, cp_size,
                                rank, softmax_scale, kernels, cu_host, steps, ctx.cu_dev)
        dq, dk, dv = dq.to(q.dtype), dkv[0].to(kv.dtype), dkv[1].to(kv.dtype)
        if packed:
            dq, dk, dv = dq.squeeze(0), dk.squeeze(0), dv.squeeze(0)
        return dq, dk, dv, None, None, None, None, None, None, None


def ring_attn(q, k, v, window_size: int, cp_group, cp_size: int, cp_local_rank: int,
              softmax_scale: Optional[float] = None, cu_seqlens=None, *, kernels=None):
    """Attention output of this rank's chunk.  ``cu_seqlens`` (host list or tensor of the
    whole pack) switches to packed ``[tokens, heads, dim]`` chunks."""
    assert cp_group is not None and cp_size is not None and cp_local_rank is not None, (
        "cp_group needs cp_size and cp_local_rank"
    )
    cu_host = None
    if cu_seqlens is not None:
        cu_host = cu_seqlens.tolist() if torch.is_tensor(cu_seqlens) else list(cu_seqlens)
        assert q.shape[0] == cu_host[-1] // cp_size, (
            "cu_seqlens does not match with sequence length per rank"
        )
    return RingSlidingWindowFunc.apply(q, k, v, int(window_size), cp_group, int(cp_size),
                                       int(cp_local_rank), softmax_scale, kernels, cu_host)
