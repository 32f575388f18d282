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

The compute is ``rank_share.blocks_forward`` / ``blocks_backward`` -- the one implementation of
a rank's blocks on the four block operators of ``ops/accum.py`` with upstream's accumulator
types (fp32 output, fp64 LSE, fp32 dq / dkv), which ``ring_rank_share_attn(ring_dtypes=True)``
runs as well; on the HIP library the accumulators are written and added to in the kernels'
epilogues.  ``kernels`` selects the primitives under the operators: the HIP library by
default; the CPU test tier passes stand-ins and runs this file over gloo.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch

from .ops.band_attn import attn_fwd
from .ops.p2p import exchange, get_group_local_to_global_rank_map
from .rank_share import (Step, _backward_two_blocks, blocks_backward, blocks_forward,
                         plan_nonvarlen, plan_varlen, ring_comm_times)


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


def band_forward(q, kv, window_size, cp_group, cp_size, rank, softmax_scale, kernels, cu_host,
                 narrow=False):
    """Forward of the band blocks of one rank on ``[batch, seq, heads, dim]`` chunks (batch 1
    around a packed chunk): returns the accumulators of
    ``ring_swa/sliding_window/nonvarlen.py:53-59`` -- fp32 output, fp64 LSE -- before their
    final cast, the device ``cu_seqlens`` of the own-chunk block (packed), the block plan and
    the received key ranges by hop.

    ``narrow=True`` (HIP library only) lets a plan of exactly two blocks -- the window no longer
    than a chunk, the common case -- run without the wide accumulators: the second block is merged
    into the first one's 16-bit output and fp32 LSE in its kernel's epilogue.  One merge, one
    rounding: the bits the fp32 / fp64 accumulators give after their final cast, without their
    extra passes over the output (the same two routes of the single-GPU emulation of a rank's
    step take 2.33 and 2.15 ms per forward + backward at 8192-token chunks, window 4096, 32 / 8
    heads)."""
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

    def landed():
        for req in reqs:
            req.wait()

    # own-chunk block while the key ranges are on the wire, then the blocks on them
    if narrow and kernels is None and len(steps) == 2:
        (_, _, _, window0, causal0), (i1, qs, _, window1, causal1) = steps
        if cu_dev is not None:
            out, lse = attn_fwd(q[0], kv[0][0], kv[1][0], softmax_scale, window0, causal0, cu_dev, cu_dev)
            out, lse = out.unsqueeze(0), lse.unsqueeze(0)
        else:
            out, lse = attn_fwd(q, kv[0], kv[1], softmax_scale, window0, causal0)
        landed()
        attn_fwd(q[:, qs], got[i1][0], got[i1][1], softmax_scale, window1, causal1,
                 accumulate_into=(out[:, qs], lse[:, :, qs]))
        return out, lse, cu_dev, steps, got
    out, lse = blocks_forward(q, kv, got, steps, softmax_scale, cu_dev, kernels, before_rest=landed)
    return out, lse, cu_dev, steps, got


def band_backward(q, kv, out, lse, do, got_list, window_size, cp_group, cp_size, rank,
                  softmax_scale, kernels, cu_host, steps, cu_dev, narrow=False):
    """Backward of the same blocks from the final ``(out, lse)``: fp32 ``dq`` and ``dkv`` of this
    rank's chunk, the contributions of later ranks included.  ``narrow=True``: a plan of two
    blocks on the HIP library sums its two dq partials inside the dQ kernel and returns 16-bit
    ``dq``; ``dkv`` is 16-bit unless later ranks contribute to it (then fp32: own gradients and
    contributions summed in fp32, in hop order, as with the wide accumulators)."""
    s = q.shape[1]
    gmap = get_group_local_to_global_rank_map(cp_group)
    kv_of = {i: kv_i for (i, *_r), kv_i in zip(steps[1:], got_list)}
    dkv_of = {i: torch.empty_like(kv_i) for i, kv_i in kv_of.items()}
    incoming = _incoming(rank, s, window_size, cp_size, cu_host)
    back = [kv.new_empty((2, kv.shape[1], ks.stop - ks.start, kv.shape[3], kv.shape[4]))
            for (_, _, ks) in incoming]
    reqs = []

    def send_back():
        # the blocks on received key ranges are done: their dKV goes back to the owners while
        # the own-chunk block runs
        sends = [(dkv_of[i], gmap[rank - i]) for (i, *_r) in steps[1:]]
        recvs = [(buf, gmap[other]) for buf, (_, other, _) in zip(back, incoming)]
        reqs.extend(exchange(sends, recvs, cp_group))

    if narrow and kernels is None and len(steps) == 2:
        i1 = steps[1][0]
        dq, dkv = _backward_two_blocks(q, kv[0], kv[1], kv_of[i1], dkv_of[i1], out, lse, do, steps,
                                       softmax_scale, cu_dev, wide=False, after_rest=send_back)
        if incoming:
            dkv = dkv.float()
    else:
        dq, dkv = blocks_backward(q, kv, kv_of, out, lse, do, steps, softmax_scale, cu_dev, dkv_of,
                                  kernels, after_rest=send_back)
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
                                                    softmax_scale, kernels, cu_host, narrow=True)
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
                                rank, softmax_scale, kernels, cu_host, steps, ctx.cu_dev,
                                narrow=True)
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
