"""One context-parallel rank's share of ring sliding-window attention, on one GPU.

The compute body of upstream's ring loops
(``ring_swa/sliding_window/nonvarlen.py:46-150`` forward, ``:182-333`` backward;
``ring_swa/sliding_window/varlen.py:56-172`` and ``:194-359``) with the P2P
exchange replaced by KV chunks the caller already holds in HBM: the rank's own
chunk plus the chunks of the ranks before it.  Per step: one band-attention
kernel on the block the window selects, LSE-merged into the running output;
backward runs one kernel call per block with the final merged ``(o, lse)`` and
accumulates ``dq`` / per-chunk ``dkv`` in fp32, as upstream does.

What is left out is exactly what needs a second GPU: moving KV forward and
KV + dKV backward around the ring.
"""
from __future__ import annotations

import math
import threading
from typing import List, Optional, Sequence, Tuple

import torch

from .ops.accum import (flash_attn_bwd_func, flash_attn_fwd_func, flash_attn_varlen_bwd_func,
                        flash_attn_varlen_fwd_func, hip_kernels)
from .ops.band_attn import attn_bwd, attn_fwd, bwd_handoff_active, bwd_workspace_bytes

Step = Tuple[int, slice, slice, Tuple[int, int], bool]


def ring_comm_times(window_size: int, seq_len: int, cp_size: int) -> int:
    """Number of KV hops a rank needs: ``min(ceil(w / S), cp_size - 1)``
    (``ring_swa/sliding_window/nonvarlen.py:46-49``)."""
    return min(math.ceil(window_size / seq_len), cp_size - 1)


def plan_nonvarlen(seq_len: int, window_size: int, cp_size: int, rank: int) -> List[Step]:
    """Blocks of one rank as ``(step, q_slice, kv_slice, (left, right), causal)``.

    Step ``i`` pairs the rank's queries with the chunk of rank ``rank - i``; the
    four block shapes are those of ``ring_swa/sliding_window/nonvarlen.py:95-150``
    (diagonal / full / lower-left corner cut / upper-right corner only).
    Wrap-around steps are dropped (``:97``).
    """
    s, w = seq_len, window_size
    plan: List[Step] = []
    whole = slice(0, s)
    for i in range(ring_comm_times(w, s, cp_size) + 1):
        if rank - i < 0:
            continue
        if i == 0:
            plan.append((0, whole, whole, (w, 0), True))
        elif (i + 1) * s <= w + 1:
            plan.append((i, whole, whole, (-1, -1), False))
        elif i * s < w + 1:
            plan.append((i, whole, whole, (w % s, s), False))
        elif (i - 1) * s < w < i * s:
            v = w % s
            plan.append((i, slice(0, v), slice(s - v, s), (0, s), False))
        else:
            raise ValueError(f"[forward] Invalid step: {i}")
    return plan


def plan_varlen(cu_seqlens: Sequence[int], seq_len: int, window_size: int, cp_size: int,
                rank: int) -> Tuple[List[int], List[Step]]:
    """Packed twin (``ring_swa/sliding_window/varlen.py:56-74,127-172``).

    Returns the rank-local ``cu_seqlens`` of the diagonal block and the plan; only
    the rank's first sequence (the one that may start on an earlier rank) has
    off-diagonal blocks, each a dense rectangle.
    """
    cu = [int(c) for c in cu_seqlens]
    s, w = seq_len, window_size
    start, end = rank * s, (rank + 1) * s
    first = min(i for i, c in enumerate(cu) if c > start)
    last = min(i for i, c in enumerate(cu) if c >= end)
    local_cu = [0] + [c - start for c in cu[first:last]] + [s]
    first_q_len = local_cu[1]
    first_kv_len = start - cu[first - 1]
    plan: List[Step] = [(0, slice(0, s), slice(0, s), (w, 0), True)]
    for i in range(1, ring_comm_times(w, s, cp_size) + 1):
        if rank - i < 0:
            continue
        if min(first_kv_len, w) > (i - 1) * s:
            vw = min(w - (i - 1) * s, 2 * s)
            vk = min(first_kv_len - (i - 1) * s, s, vw)
            vq = min(first_q_len, vw)
            plan.append((i, slice(0, vq), slice(s - vk, s), (vw - vq, s), False))
    return local_cu, plan


class RankShareFunc(torch.autograd.Function):
    """Dense tensors ``[batch, seq, heads, dim]``; ``prev_kv[i - 1]`` is the stacked
    ``[2, batch, seq, kv_heads, dim]`` chunk of rank ``rank - i``."""

    @staticmethod
    def forward(ctx, q, k, v, window_size, cp_size, rank, softmax_scale, ring_dtypes, one_pass,
                *prev_kv):
        b, s, hq, d = q.shape
        if softmax_scale is None:
            softmax_scale = d ** (-0.5)
        plan = plan_nonvarlen(s, window_size, cp_size, rank)
        for (i, _, _, _, _) in plan:
            assert i == 0 or i <= len(prev_kv), f"step {i} needs the chunk of rank {rank - i}"
        out, lse = _forward_blocks(q, k, v, prev_kv, plan, softmax_scale, None, ring_dtypes,
                                   one_pass)
        ctx.save_for_backward(q, k, v, out, lse, *prev_kv)
        ctx.plan, ctx.scale, ctx.ring_dtypes, ctx.one_pass = plan, softmax_scale, ring_dtypes, one_pass
        return out

    @staticmethod
    def backward(ctx, do):
        q, k, v, out, lse, *prev_kv = ctx.saved_tensors
        grads = _backward_blocks(q, k, v, prev_kv, out, lse, do, ctx.plan, ctx.scale, None,
                                 ctx.ring_dtypes, ctx.one_pass)
        return (grads[0], grads[1], grads[2], None, None, None, None, None, None, *grads[3:])


_CU_CACHE = {}


def _device_cu(local_cu: Sequence[int], device: torch.device) -> torch.Tensor:
    """int32 device copy of a rank's local ``cu_seqlens``, cached: a training loop calls
    every layer with the same packing, and each fresh host-to-device copy of a Python list
    is a blocking call that stops the host from running ahead of the GPU."""
    key = (tuple(local_cu), device.index)
    t = _CU_CACHE.get(key)
    if t is None:
        if len(_CU_CACHE) >= 256:
            _CU_CACHE.clear()
        t = _CU_CACHE[key] = torch.tensor(local_cu, dtype=torch.int32, device=device)
    return t


class RankShareVarlenFunc(torch.autograd.Function):
    """Packed tensors ``[tokens, heads, dim]``; ``prev_kv[i - 1]`` is ``[2, tokens, kv_heads, dim]``."""

    @staticmethod
    def forward(ctx, q, k, v, window_size, cu_host, cp_size, rank, softmax_scale, ring_dtypes,
                *prev_kv):
        s, hq, d = q.shape
        if softmax_scale is None:
            softmax_scale = d ** (-0.5)
        local_cu, plan = plan_varlen(cu_host, s, window_size, cp_size, rank)
        cu_dev = _device_cu(local_cu, q.device)
        q4, k4, v4 = q.unsqueeze(0), k.unsqueeze(0), v.unsqueeze(0)
        prev4 = [p.unsqueeze(1) for p in prev_kv]
        out, lse = _forward_blocks(q4, k4, v4, prev4, plan, softmax_scale, cu_dev, ring_dtypes)
        out, lse = out.squeeze(0), lse.squeeze(0)
        ctx.save_for_backward(q, k, v, out, lse, cu_dev, *prev_kv)
        ctx.plan, ctx.scale, ctx.ring_dtypes = plan, softmax_scale, ring_dtypes
        return out

    @staticmethod
    def backward(ctx, do):
        q, k, v, out, lse, cu_dev, *prev_kv = ctx.saved_tensors
        prev4 = [p.unsqueeze(1) for p in prev_kv]
        grads = _backward_blocks(q.unsqueeze(0), k.unsqueeze(0), v.unsqueeze(0), prev4,
                                 out.unsqueeze(0), lse.unsqueeze(0), do.unsqueeze(0), ctx.plan,
                                 ctx.scale, cu_dev, ctx.ring_dtypes)
        dprev = [g.squeeze(1) for g in grads[3:]]
        return (grads[0].squeeze(0), grads[1].squeeze(0), grads[2].squeeze(0), None, None, None,
                None, None, None, *dprev)


_SIDE_STREAMS = threading.local()  # .by_device: {device index: stream}; gone with its thread


def _fork(device: torch.device) -> "torch.cuda.Stream":
    """Side stream (default priority, one per device and host thread) ordered after the
    current stream.

    The blocks of one step are independent until they are merged, and each launch alone
    leaves compute units idle in its tail (few, unequal work groups), so the diagonal
    block runs on the caller's stream and the other blocks on this one; ``_join``
    orders the caller's stream after them again.  Tensors used on the side stream are
    allocated on the caller's stream before the fork (or marked with ``record_stream``), so
    the caching allocator hands their memory back to the caller's stream only."""
    by_device = getattr(_SIDE_STREAMS, "by_device", None)
    if by_device is None:
        by_device = _SIDE_STREAMS.by_device = {}
    side = by_device.get(device.index)
    if side is None:
        side = by_device[device.index] = torch.cuda.Stream(device)
    side.wait_stream(torch.cuda.current_stream(device))
    return side


def _join(side: "torch.cuda.Stream", device: torch.device) -> None:
    torch.cuda.current_stream(device).wait_stream(side)


def blocks_forward(q, kv, kv_of, plan, scale, local_cu, kernels=None, before_rest=None):
    """The planned blocks of one rank through the accumulating block operators -- upstream's flow
    and accumulator types (``ring_swa/sliding_window/nonvarlen.py:53-59, 95-154``): fp32 output
    and fp64 LSE, every block merged into its row range; returns the accumulators before their
    final cast.  ``kv`` is the rank's own chunk, stacked ``[2, batch, seq, kv_heads, dim]`` or the pair ``(k, v)``,
    ``kv_of[i]`` the stacked key range the block of step ``i`` reads (of rank ``rank - i``:
    received by a ring, sliced from a held chunk by the single-GPU emulation), ``local_cu`` the
    device ``cu_seqlens`` of the own-chunk block of a packed chunk (batch 1).  ``before_rest`` is
    called between the own-chunk block and the others (a ring waits for its receives there).
    This one function is what ``ring_rank_share_attn(ring_dtypes=True)``, plans of three and
    more blocks and the ring over a ``cp_group`` (``ring_swa/ring.py``) all run; on the HIP library
    the operators work in the kernels' epilogues: the own-chunk block writes the accumulators
    (they are never filled with the merge identity), the others merge into them, no temporary,
    no merge launch."""
    assert plan and plan[0][0] == 0, "the diagonal block comes first: it covers every row"
    b, s, hq, _ = q.shape
    out = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    lse = torch.empty((b, hq, s), dtype=torch.float64, device=q.device)
    (_, _, _, window0, causal0) = plan[0]
    if local_cu is not None:
        flash_attn_varlen_fwd_func(q, kv, scale, window0, local_cu, local_cu, None, None, causal0,
                                   out, lse, kernels=kernels, fresh=True)
    else:
        flash_attn_fwd_func(q, kv, scale, window0, causal0, out, lse, kernels=kernels, fresh=True)
    if before_rest is not None:
        before_rest()
    for (i, qs, _, window, causal) in plan[1:]:
        flash_attn_fwd_func(q[:, qs], kv_of[i], scale, window, causal, out[:, qs], lse[:, :, qs],
                            kernels=kernels)
    return out, lse


def blocks_backward(q, kv, kv_of, out, lse, do, plan, scale, local_cu, dkv_of, kernels=None,
                    after_rest=None):
    """Backward of the same blocks from the final 16-bit ``out`` and fp32 ``lse``
    (``ring_swa/sliding_window/nonvarlen.py:203-206, 233-321``): returns fp32 ``dq`` and fp32
    ``dkv`` of the own chunk; the gradients of the key range of step ``i`` are written, in the
    keys' type, into ``dkv_of[i]`` (a ring sends them back to the keys' owner; the emulation
    passes views of the held chunks' gradients).  The blocks on other ranks' keys run first and
    ``after_rest`` is called before the own-chunk block, so that a ring has their gradients on
    the wire while it computes its largest block.  ``dq`` is never zero-filled: the first block
    writes its rows (every later block's rows lie inside them: the plans' row ranges are
    prefixes that shrink with the hop), the rows beyond get zeros, every further block adds."""
    assert plan and plan[0][0] == 0
    if len(plan) == 2 and (kernels is None or kernels is hip_kernels()) and q.is_cuda:
        # exactly one other block, on the HIP library: the two-stream schedule (same sums)
        i1 = plan[1][0]
        return _backward_two_blocks(q, kv[0], kv[1], kv_of[i1], dkv_of[i1], out, lse, do, plan,
                                    scale, local_cu, wide=True, after_rest=after_rest)
    dq = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    dkv = torch.empty((2,) + tuple(kv[0].shape), dtype=torch.float32, device=q.device)
    first = True
    covered = q.shape[1]
    for (i, qs, _, window, causal) in plan[1:]:
        q0, q1, _ = qs.indices(q.shape[1])
        assert q0 == 0 and q1 <= covered, "row ranges of the plan must be shrinking prefixes"
        if first:
            dq[:, q1:].zero_()
            covered = q1
        flash_attn_bwd_func(q[:, qs], kv_of[i], out[:, qs], lse[:, :, qs], do[:, qs], dq[:, qs],
                            dkv_of[i], scale, window, causal, kernels=kernels,
                            accumulate_dq=not first)
        first = False
    if after_rest is not None:
        after_rest()
    (_, _, _, window0, causal0) = plan[0]
    if local_cu is not None:
        flash_attn_varlen_bwd_func(q, kv, out, lse, do, dq, dkv, local_cu, local_cu, None, None,
                                   scale, window0, causal0, kernels=kernels,
                                   accumulate_dq=not first)
    else:
        flash_attn_bwd_func(q, kv, out, lse, do, dq, dkv, scale, window0, causal0, kernels=kernels,
                            accumulate_dq=not first)
    return dq, dkv


def _forward_blocks_accum(q, k, v, prev_kv, plan, scale, local_cu):
    """``blocks_forward`` on key ranges sliced from the held chunks of earlier ranks."""
    kv_of = {i: prev_kv[i - 1][:, :, ks] for (i, _, ks, _, _) in plan[1:]}
    out, lse = blocks_forward(q, (k, v), kv_of, plan, scale, local_cu)
    return out.to(q.dtype), lse.float()


def _one_pass(q, k, v, prev_kv, plan, local_cu):
    """Can the rank's two blocks be computed as ONE band over the previous chunk's tail
    followed by the own chunk?  Yes when the second block is the previous chunk's corner (window
    shorter than a chunk) and the previous chunk lies like the own chunk in memory: the kernels
    then take the two row ranges where they are (``second=`` of ``attn_fwd`` / ``attn_bwd``).
    The tail is the window rounded up to the 256 rows the kernels want the first range to be a
    multiple of; the rows beyond the window are masked like any key too far back.  Returns
    ``(window, tail_k, tail_v, tail_rows)`` or None."""
    if local_cu is not None or len(plan) != 2:
        return None
    (_, _, _, (w, _), _), (i1, qs, ks, window1, causal1) = plan
    s = q.shape[1]
    if i1 != 1 or causal1 or window1 != (0, s) or not (0 < w < s):
        return None
    tail = -(-w // 256) * 256
    if (qs.start, qs.stop) != (0, w) or (ks.start, ks.stop) != (s - w, s) or tail > s:
        return None
    kk, vv = prev_kv[0][0][:, s - tail:], prev_kv[0][1][:, s - tail:]
    # (the kernels apply the first range's strides to both; a stride over one element is unused)
    used = [d for d in range(4) if k.shape[d] > 1]
    if any(kk.stride(d) != k.stride(d) or vv.stride(d) != v.stride(d) for d in used):
        return None
    return w, kk, vv, tail


def _forward_blocks(q, k, v, prev_kv, plan, scale, local_cu, ring_dtypes, one_pass=True):
    """Run the planned blocks and merge them.  Dense 4-d tensors (batch 1 when packed)."""
    assert plan and plan[0][0] == 0, "the diagonal block comes first: it covers every row"
    one = _one_pass(q, k, v, prev_kv, plan, local_cu) if one_pass and not ring_dtypes else None
    if one is not None:
        # One band over [tail of the previous chunk | own chunk]: row i sees the w + 1 keys that
        # end at its own position, wherever the chunk boundary falls -- the sum the two blocks
        # and their merge compute, in one launch, with uniform work per block and no rounding of
        # a partial output in between (2.10 -> 2.02 ms per step at 8192-token chunks, window
        # 4096; two launches and a merge remain for every other shape and for ring_dtypes).
        w, kk, vv, _ = one
        return attn_fwd(q, kk, vv, scale, (w, 0), True, second=(k, v))
    if ring_dtypes or len(plan) > 2:
        # With two blocks the 16-bit running output is merged once and rounded once, the same
        # bits as the fp32 accumulator gives; from three blocks on every further merge would
        # add a rounding the reference does not have, so its accumulators are used.
        return _forward_blocks_accum(q, k, v, prev_kv, plan, scale, local_cu)
    # Own-chunk block first, then the previous-chunk block merged into its rows in the
    # forward kernel's epilogue (same bits as a separate merge).  One stream: two forward
    # launches side by side take longer than one after the other on this hardware (552 against
    # 385 + 130 us at 8192-token chunks, window 4096), and the merge launch goes away.
    (_, _, _, window, causal) = plan[0]
    if local_cu is not None:
        out, lse = attn_fwd(q[0], k[0], v[0], scale, window, causal, local_cu, local_cu)
        out, lse = out.unsqueeze(0), lse.unsqueeze(0)
    else:
        out, lse = attn_fwd(q, k, v, scale, window, causal)
    for (i, qs, ks, window, causal) in plan[1:]:
        kk, vv = prev_kv[i - 1][0], prev_kv[i - 1][1]
        attn_fwd(q[:, qs], kk[:, ks], vv[:, ks], scale, window, causal,
                 accumulate_into=(out[:, qs], lse[:, :, qs]))
    return out, lse


def _backward_blocks(q, k, v, prev_kv, out, lse, do, plan, scale, local_cu, ring_dtypes=False,
                     one_pass=True):
    if do.stride(-1) != 1:
        do = do.contiguous()
    assert plan and plan[0][0] == 0
    if len(plan) == 1 and not ring_dtypes:
        # the own-chunk block alone (rank 0, or a window that ends inside the chunk for a pack
        # whose first sequence starts in it): 16-bit gradients straight from the kernels
        dq, dkv = torch.empty_like(q), torch.empty((2,) + tuple(k.shape), dtype=k.dtype, device=k.device)
        (_, _, _, window, causal) = plan[0]
        if local_cu is not None:
            flash_attn_varlen_bwd_func(q, (k, v), out, lse, do, dq, dkv, local_cu,
                                       local_cu, None, None, scale, window, causal)
        else:
            flash_attn_bwd_func(q, (k, v), out, lse, do, dq, dkv, scale, window, causal)
        return (dq, dkv[0], dkv[1], *[torch.zeros_like(kv) for kv in prev_kv])
    if len(plan) == 2 and not ring_dtypes:
        one = _one_pass(q, k, v, prev_kv, plan, local_cu) if one_pass else None
        if one is not None:
            return _backward_one_pass(q, k, v, prev_kv, out, lse, do, one, scale)
        # (the previous chunk's dK / dV are zeroed whole: one contiguous fill is faster than a
        # strided one of half the size)
        dprev = [torch.zeros_like(kv) for kv in prev_kv]
        (i1, _, ks, _, _) = plan[1]
        dq, dkv = _backward_two_blocks(q, k, v, prev_kv[i1 - 1][:, :, ks], dprev[i1 - 1][:, :, ks],
                                       out, lse, do, plan, scale, local_cu)
        return (dq, dkv[0], dkv[1], *dprev)
    # one block, three and more, or upstream's accumulator types asked for: the accumulating
    # flow of upstream's backward on the block operators; the previous chunks' gradients are what
    # a ring would send back (zero outside the key ranges the blocks read)
    dprev = [torch.zeros_like(kv) for kv in prev_kv]
    kv_of = {i: prev_kv[i - 1][:, :, ks] for (i, _, ks, _, _) in plan[1:]}
    dkv_of = {i: dprev[i - 1][:, :, ks] for (i, _, ks, _, _) in plan[1:]}
    dq, dkv = blocks_backward(q, (k, v), kv_of, out, lse, do, plan, scale, local_cu,
                              dkv_of)
    return (dq.to(q.dtype), dkv[0].to(k.dtype), dkv[1].to(v.dtype), *dprev)


def _backward_one_pass(q, k, v, prev_kv, out, lse, do, one, scale):
    """Backward of the one-band forward: statistics, dQ and dK/dV launches on the caller's
    stream; the gradients of the previous chunk's tail land in their rows of its (zeroed)
    gradient.

    One stream: each of the two big launches fills every compute unit by itself (even blocks,
    many of them), and side by side on two streams they take longer than one after the other
    (2.01-2.04 against 1.95-1.97 ms per step at 8192-token chunks, window 4096; dQ ahead of
    dK/dV measured 0.5 % better than the other order)."""
    PREP, DKDV, DQ = 1, 2, 4
    w, kk, vv, tail = one
    s = q.shape[1]
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    dprev = [torch.zeros_like(kv) for kv in prev_kv]
    dkk, dvv = dprev[0][0][:, s - tail:], dprev[0][1][:, s - tail:]
    # (sized for the route attn_bwd will pick: handoff=None on both sides)
    ws = torch.empty(bwd_workspace_bytes(q, kk, second_rows=s, window_size=(w, 0), causal=True,
                                         handoff=None), dtype=torch.uint8, device=q.device)
    handed = bwd_handoff_active(q, kk, second_rows=s, window_size=(w, 0), causal=True)
    # the dQ kernel of the hand-off route reads what the dK/dV kernel stored
    for phases in ((PREP, DKDV, DQ) if handed else (PREP, DQ, DKDV)):
        attn_bwd(q, kk, vv, out, lse, do, dq, dkk, dvv, scale, (w, 0), True, workspace=ws,
                 phases=phases, second=(k, v, dk, dv))
    return (dq, dk, dv, *dprev)


def _backward_two_blocks(q, k, v, kv1, dkv1, out, lse, do, plan, scale, local_cu, wide=False,
                         after_rest=None):
    """Own-chunk block + one block on another rank's key range ``kv1`` (stacked, already sliced;
    its gradients go to ``dkv1`` in the keys' type), on two streams, with dq summed inside the dQ
    kernel instead of in separate passes.  The other block writes its dQ first (side stream); the
    own-chunk dQ kernel, ordered after it, adds to it: fp32 sum of the two 16-bit partials --
    rounded once into a 16-bit ``dq``, or kept in the fp32 ``dq`` / ``dk`` / ``dv`` of ``wide=True``
    (the ring loops' accumulators): bit for bit what the fp32 accumulator of
    ring_swa/sliding_window/nonvarlen.py:203, 318-321 yields for two blocks, either way.
    ``after_rest`` is called on the side stream once the other block's launches are enqueued
    there (a ring starts sending its dKV back from that stream).  Returns ``dq`` and the stacked
    ``dkv`` of the own chunk.

    Launch order (measured; each variant below costs 1-6 % of the step): the side stream
    gets its launches first and runs the other block's dQ kernel before its dK/dV kernel.  The
    own-chunk dQ kernel then never waits (what it needs is finished long before the own-chunk
    dK/dV kernel is), and the other block's dK/dV blocks -- few, of very unequal length -- fill
    the compute units that the short blocks of the own-chunk dK/dV launch and the tail of the
    own-chunk dQ launch leave idle.  Delaying the side stream's kernels (zero fills on it,
    own-chunk launches ahead of it) lets the own-chunk dK/dV launch take every compute unit
    first and loses that packing."""
    PREP, DKDV, DQ = 1, 2, 4
    (_, _, _, window0, causal0), (i1, qs, ks, window1, causal1) = plan
    # Of dq only the rows outside the other block are zeroed (the own-chunk dQ kernel adds to
    # every row; the other block's kernel writes its own).
    q0, q1, _ = qs.indices(q.shape[1])
    gdt = torch.float32 if wide else q.dtype
    dq = torch.empty(q.shape, dtype=gdt, device=q.device)
    dkv = torch.empty((2,) + tuple(k.shape), dtype=gdt, device=q.device)
    dk, dv = dkv[0], dkv[1]
    dq[:, :q0].zero_()
    dq[:, q1:].zero_()
    # (the launches below run dQ ahead of dK/dV, which the dS hand-off cannot: handoff=False)
    if local_cu is not None:
        need = bwd_workspace_bytes(q[0], k[0], local_cu, local_cu)
    else:
        need = bwd_workspace_bytes(q, k)
    ws = torch.empty(need, dtype=torch.uint8, device=q.device)
    ws_prev = torch.empty(bwd_workspace_bytes(q[:, qs], kv1[0]), dtype=torch.uint8, device=q.device)

    def own(phases, accumulate):
        if local_cu is not None:
            attn_bwd(q[0], k[0], v[0], out[0], lse[0], do[0], dq[0], dk[0], dv[0], scale, window0,
                     causal0, local_cu, local_cu, workspace=ws, phases=phases,
                     dq_accumulate=accumulate, handoff=False)
        else:
            attn_bwd(q, k, v, out, lse, do, dq, dk, dv, scale, window0, causal0, workspace=ws,
                     phases=phases, dq_accumulate=accumulate, handoff=False)

    def prev(phases):
        attn_bwd(q[:, qs], kv1[0], kv1[1], out[:, qs], lse[:, :, qs], do[:, qs], dq[:, qs],
                 dkv1[0], dkv1[1], scale, window1, causal1, workspace=ws_prev,
                 phases=phases, dq_accumulate=False, handoff=False)

    side = _fork(q.device)
    with torch.cuda.stream(side):
        prev(PREP | DQ)
        dq_prev_done = torch.cuda.Event()
        dq_prev_done.record(side)
        prev(DKDV)
        if after_rest is not None:
            after_rest()
    own(PREP | DKDV, False)
    torch.cuda.current_stream(q.device).wait_event(dq_prev_done)
    own(DQ, True)
    _join(side, q.device)
    return dq, dkv


def ring_rank_share_attn(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    prev_kv: Sequence[torch.Tensor],
    window_size: int,
    cp_size: int,
    cp_local_rank: int,
    softmax_scale: Optional[float] = None,
    *,
    ring_dtypes: bool = False,
    one_pass: bool = True,
) -> torch.Tensor:
    """Attention output of rank ``cp_local_rank`` for its chunk ``q, k, v``
    (``[batch, seq, heads, dim]``), given ``prev_kv[i - 1] = stack([k, v])`` of rank
    ``cp_local_rank - i``.  Differentiable w.r.t. ``q, k, v`` and every ``prev_kv``
    entry (the gradient a real ring would send back).  ``ring_dtypes=True`` keeps the
    running output in fp32 and the running LSE in fp64 as upstream does.  ``one_pass=False``
    keeps upstream's block structure -- own-chunk block, previous-chunk block, LSE merge
    (``ring_swa/sliding_window/nonvarlen.py:95-154``) -- where the default computes the two as
    one band over both key ranges (window shorter than a chunk)."""
    assert q.shape[1] == k.shape[1] == v.shape[1], "Sequence length must be the same"
    return RankShareFunc.apply(q, k, v, int(window_size), int(cp_size), int(cp_local_rank),
                               softmax_scale, bool(ring_dtypes), bool(one_pass), *prev_kv)


def ring_rank_share_attn_varlen(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    prev_kv: Sequence[torch.Tensor],
    window_size: int,
    cu_seqlens,
    cp_size: int,
    cp_local_rank: int,
    softmax_scale: Optional[float] = None,
    *,
    ring_dtypes: bool = False,
) -> torch.Tensor:
    """Packed twin: ``q, k, v`` are the rank's ``[tokens, heads, dim]`` slice of the
    pack and ``cu_seqlens`` the cumulative lengths of the WHOLE pack (a host list or a
    tensor, read once on the host to lay out the blocks)."""
    cu_host = cu_seqlens.tolist() if torch.is_tensor(cu_seqlens) else list(cu_seqlens)
    assert q.shape[0] == cu_host[-1] // cp_size, (
        "cu_seqlens does not match with sequence length per rank"
    )
    return RankShareVarlenFunc.apply(q, k, v, int(window_size), cu_host, int(cp_size),
                                     int(cp_local_rank), softmax_scale, bool(ring_dtypes), *prev_kv)
