"""Streaming-LLM attention (sink tokens + sliding window) over a context-parallel group.

Same result as the single-process functions of ``streaming_llm.py`` on the whole sequence:
every query sees the ``window_size + 1`` keys of its band and, beyond the band, the first
``num_sink_tokens`` tokens of its own sequence.  Takes the place of the upstream ring
(``ring_swa/streaming_llm/nonvarlen.py:19-397``, ``varlen.py:19-473``), which broadcasts one
sink token from rank 0 to everybody, merges it analytically into every row and reduces /
all-to-alls the sink gradients.  Here:

* the band part is the sliding-window ring of ``ring.py`` unchanged (sink tokens inside the
  window are ordinary band keys);
* the part beyond the band is one more block per rank -- the rank's rows against the sink rows
  of their sequence, visible where the sink lies left of the window (an explicit diagonal shift
  of the block mask: ``j <= position(i) - window_size - 1``) -- merged into the same
  accumulators.  A rank whose chunk starts inside a sequence fetches that sequence's sink rows
  from the rank(s) that hold them, point to point (``num_sink_tokens`` rows, not a collective);
  sequences that start inside the chunk have their sinks at hand;
* in the backward the block's dK / dV of fetched sink rows go straight back to their owner,
  which adds them in fp32 in rank order.

Who needs which rows from whom follows from ``(seq_len, cp_size, window_size,
num_sink_tokens)`` and the pack's ``cu_seqlens`` alone, so every rank computes every rank's
plan and no request messages exist.  Sinks are per sequence (upstream's packed ring uses the
pack's first token for all sequences and requires them to start alike).
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from .ops.accum import hip_kernels
from .ops.p2p import exchange, get_group_local_to_global_rank_map
from .ring import band_backward, band_forward


def sink_plan(rank: int, seq_len: int, window_size: int, n_sink: int,
              cu: Sequence[int]) -> List[dict]:
    """The segments of rank ``rank``'s chunk (one per sequence that has rows in it) some row of
    which sees a sink from beyond the window.  Per segment: ``rows`` (local row slice), ``p0``
    (position of its first row inside its sequence), ``n`` (sink rows that can matter) and
    ``pieces``: ``(owner rank, owner's local row slice, offset among the n sink rows)``."""
    lo, hi = rank * seq_len, (rank + 1) * seq_len
    segs = []
    for g0, g1 in zip(cu[:-1], cu[1:]):
        x0, x1 = max(g0, lo), min(g1, hi)
        if x0 >= x1:
            continue
        p0 = x0 - g0
        # a row at position p sees sink j from beyond the window iff j < p - window_size
        n = min(n_sink, g1 - g0, p0 + (x1 - x0) - 1 - window_size)
        if n <= 0:
            continue
        pieces = []
        for owner in range(g0 // seq_len, (g0 + n - 1) // seq_len + 1):
            y0, y1 = max(g0, owner * seq_len), min(g0 + n, (owner + 1) * seq_len)
            pieces.append((owner, slice(y0 - owner * seq_len, y1 - owner * seq_len), y0 - g0))
        segs.append({"rows": slice(x0 - lo, x1 - lo), "p0": p0, "n": n, "pieces": pieces})
    return segs


def _serves(rank: int, seq_len: int, window_size: int, n_sink: int, cu: Sequence[int],
            cp_size: int):
    """``(later rank, local row slice)`` for every piece of this rank's rows that a later rank
    fetches, in the order that rank lists them."""
    out = []
    for other in range(rank + 1, cp_size):
        for seg in sink_plan(other, seq_len, window_size, n_sink, cu):
            for owner, rows, _ in seg["pieces"]:
                if owner == rank:
                    out.append((other, rows))
    return out


class RingStreamingLLMFunc(torch.autograd.Function):
    """Dense ``[batch, seq, heads, dim]`` chunks (``cu_host`` None), or packed ``[tokens, heads,
    dim]`` chunks with ``cu_host`` = cumulative lengths of the whole pack (host list)."""

    @staticmethod
    def forward(ctx, q, k, v, window_size, n_sink, cp_group, cp_size, rank, softmax_scale,
                kernels, cu_host):
        K = kernels or hip_kernels()
        packed = cu_host is not None
        if packed:
            q, k, v = q.unsqueeze(0), k.unsqueeze(0), v.unsqueeze(0)
        b, s, hq, d = q.shape
        if softmax_scale is None:
            softmax_scale = d ** (-0.5)
        cu = list(cu_host) if packed else [0, s * cp_size]
        kv = torch.stack([k, v], dim=0)
        gmap = get_group_local_to_global_rank_map(cp_group)

        # sink rows: fetched pieces arrive first (a handful of rows), then everything is local
        segs = sink_plan(rank, s, window_size, n_sink, cu)
        recvs, landing = [], []
        for seg in segs:
            for owner, rows, off in seg["pieces"]:
                if owner != rank:
                    buf = kv.new_empty((2, b, rows.stop - rows.start, kv.shape[3], d))
                    recvs.append((buf, gmap[owner]))
                    landing.append((seg, off, buf))
        sends = [(kv[:, :, rows].contiguous(), gmap[other])
                 for other, rows in _serves(rank, s, window_size, n_sink, cu, cp_size)]
        for req in exchange(sends, recvs, cp_group):
            req.wait()
        sink_kv = []
        for seg in segs:
            parts = []
            for owner, rows, off in seg["pieces"]:
                if owner == rank:
                    parts.append(kv[:, :, rows])
                else:
                    parts.append(next(buf for (sg, o, buf) in landing if sg is seg and o == off))
            sink_kv.append(torch.cat(parts, dim=2) if len(parts) > 1 else parts[0].contiguous())

        out, lse, cu_dev, steps, got = band_forward(q, kv, window_size, cp_group, cp_size, rank,
                                                    softmax_scale, kernels, cu_host)
        for seg, skv in zip(segs, sink_kv):
            rows = seg["rows"]
            o_s, l_s = K.fwd(q[:, rows], skv[0], skv[1], softmax_scale, (-1, 0), False,
                             mask_shift=seg["p0"] - (window_size + 1))
            K.merge(out[:, rows], lse[:, :, rows], o_s, l_s)
        out = out.to(q.dtype)
        lse = lse.to(torch.float32)

        ctx.save_for_backward(q, kv, out, lse, *(got[i] for (i, *_rest) in steps[1:]), *sink_kv)
        ctx.n_got = len(steps) - 1
        ctx.cu_dev = cu_dev
        ctx.meta = (window_size, n_sink, cp_group, cp_size, rank, softmax_scale, kernels, cu_host,
                    steps, segs, cu)
        return out.squeeze(0) if packed else out

    @staticmethod
    def backward(ctx, do):
        q, kv, out, lse, *rest = ctx.saved_tensors
        got_list, sink_kv = rest[:ctx.n_got], rest[ctx.n_got:]
        (window_size, n_sink, cp_group, cp_size, rank, softmax_scale, kernels, cu_host, steps,
         segs, cu) = ctx.meta
        K = kernels or hip_kernels()
        packed = cu_host is not None
        if packed:
            do = do.unsqueeze(0)
        if do.stride(-1) != 1:
            do = do.contiguous()
        s = q.shape[1]
        gmap = get_group_local_to_global_rank_map(cp_group)

        dq, dkv = band_backward(q, kv, out, lse, do, got_list, window_size, cp_group, cp_size,
                                rank, softmax_scale, kernels, cu_host, steps, ctx.cu_dev)
        # the blocks on sink rows: dq stays here, dK / dV of fetched rows go back to their owner
        sends = []
        for seg, skv in zip(segs, sink_kv):
            rows = seg["rows"]
            dq_s = torch.empty_like(q[:, rows])
            dkv_s = torch.empty_like(skv)
            K.bwd(q[:, rows], skv[0], skv[1], out[:, rows], lse[:, :, rows], do[:, rows], dq_s,
                  dkv_s[0], dkv_s[1], softmax_scale, (-1, 0), False,
                  mask_shift=seg["p0"] - (window_size + 1))
            dq[:, rows] += dq_s
            for owner, own_rows, off in seg["pieces"]:
                piece = dkv_s[:, :, off:off + (own_rows.stop - own_rows.start)]
                if owner == rank:
                    dkv[:, :, own_rows] += piece
                else:
                    sends.append((piece.contiguous(), gmap[owner]))
        serves = _serves(rank, s, window_size, n_sink, cu, cp_size)
        back = [kv.new_empty((2, kv.shape[1], rows.stop - rows.start, kv.shape[3], kv.shape[4]))
                for _, rows in serves]
        recvs = [(buf, gmap[other]) for buf, (other, _) in zip(back, serves)]
        for req in exchange(sends, recvs, cp_group):
            req.wait()
        for buf, (_, rows) in zip(back, serves):  # rank order: a fixed order of the fp32 sums
            dkv[:, :, rows] += buf

        dq, dk, dv = dq.to(q.dtype), dkv[0].to(kv.dtype), dkv[1].to(kv.dtype)
        if packed:
            dq, dk, dv = dq.squeeze(0), dk.squeeze(0), dv.squeeze(0)
        return dq, dk, dv, None, None, None, None, None, None, None, None


def ring_slm_attn(q, k, v, window_size: int, cp_group, cp_size: int, cp_local_rank: int,
                  softmax_scale: Optional[float] = None, cu_seqlens=None, *,
                  num_sink_tokens: int = 1, kernels=None):
    """Attention output of this rank's chunk.  ``cu_seqlens`` (host list or tensor of the whole
    pack) switches to packed ``[tokens, heads, dim]`` chunks."""
    assert cp_group is not None and cp_size is not None and cp_local_rank is not None, (
        "cp_group needs cp_size and cp_local_rank"
    )
    assert num_sink_tokens >= 0
    cu_host = None
    if cu_seqlens is not None:
        cu_host = cu_seqlens.tolist() if torch.is_tensor(cu_seqlens) else list(cu_seqlens)
        assert q.shape[0] == cu_host[-1] // cp_size, (
            "cu_seqlens does not match with sequence length per rank"
        )
    return RingStreamingLLMFunc.apply(q, k, v, int(window_size), int(num_sink_tokens), cp_group,
                                      int(cp_size), int(cp_local_rank), softmax_scale, kernels,
                                      cu_host)
