"""Block operators of the ring loops: one attention block merged into running accumulators
(forward), one block's gradients into caller buffers (backward).

Names, positional order and in-place behaviour of the four operators of the upstream package
(``ring_swa/ops/attn.py:12-60, 63-126, 129-160, 163-196``), so a ring loop written against
them runs on this package unchanged:

* ``kv`` is the stacked pair ``[2, batch, seq, kv_heads, dim]`` (a caller that holds ``k`` and
  ``v`` separately may pass the tuple ``(k, v)`` and save the copy);
* forward: the block's ``(out, lse)`` is merged into ``global_attn_out`` (fp32 upstream) and
  ``global_softmax_lse`` (fp64 upstream, ``[batch, heads, seq]``) in place, whose start
  state ``(0, -inf)`` is the merge identity; sliced views (``[:, :v]``) are fine;
* backward: ``dq`` and ``dkv`` are overwritten with this block's gradients (in the
  tensors' 16-bit type), computed from the caller's final ``o`` / ``softmax_lse``.

More query rows than keys (``q.shape[1] > kv.shape[2]``) with a window: upstream runs the
leading ``Sq - Sk`` rows against all keys and the last ``Sk`` rows with the window
(``ops/attn.py:38-60, 90-126``).  That is the bottom-right aligned window rule of the kernels
whenever the right bound reaches the last key from every row (``right >= Sq - 1``, as in every
call the ring makes: ``right = seq_len``), so one kernel call serves it; other right bounds
take the same two-part route as upstream.

Every operator takes ``kernels=``: the five primitives it is built on (block forward /
backward, dense and packed, and the merge).  The default is the HIP library; a host-side
test of the ring logic passes stand-ins that work on CPU tensors.

Keyword-only additions.  ``fresh=True`` (forward): the accumulators hold nothing yet -- not
even the merge identity -- and the block is written into them; a ring loop starts its
accumulators that way instead of filling them with ``(0, -inf)`` first.  ``accumulate_dq`` /
``accumulate_dkv`` (backward): ``dq`` / ``dkv`` are the loop's fp32 accumulators
(``ring_swa/sliding_window/nonvarlen.py:203-206``) and the block's 16-bit gradients are added to
them, the ``dq += dq_i`` / ``dkv += dkv_i`` of ``:318-321``; without the flags a buffer of either
type is overwritten.  On the HIP library all of this happens in the kernels' epilogues
(``accumulate_into`` / ``into`` of ``attn_fwd``, fp32 buffers of ``attn_bwd``): no temporary
``(out, lse)``, no merge launch, no elementwise pass; stand-in kernels get the unfused flow.
"""
from __future__ import annotations

from types import SimpleNamespace
from typing import Optional, Tuple

import torch

_HIP = None


def hip_kernels() -> SimpleNamespace:
    """The five primitives on the HIP library (``rswa_attn_fwd`` / ``rswa_attn_bwd`` /
    ``rswa_merge_attn_out`` behind them)."""
    global _HIP
    if _HIP is None:
        from . import band_attn, lse_merge

        _HIP = SimpleNamespace(
            fwd=band_attn.wrapped_flash_attn_fwd,
            fwd_varlen=band_attn.wrapped_flash_attn_fwd_varlen,
            bwd=band_attn.wrapped_flash_attn_bwd,
            bwd_varlen=band_attn.wrapped_flash_attn_bwd_varlen,
            merge=lse_merge.merge_attn_out,
            # the kernels' own epilogues in place of temporaries + merge / elementwise sums
            fwd_fused=band_attn.attn_fwd,
            bwd_fused=band_attn.attn_bwd,
        )
    return _HIP


def _fwd_into(K, q, k, v, scale, window, causal, cu_q, cu_k, out_acc, lse_acc, fresh):
    """One block into the accumulators (4-d views; batch 1 around a pack)."""
    packed = cu_q is not None
    fused = getattr(K, "fwd_fused", None)
    if fused is not None:
        if packed:
            q, k, v, out_acc, lse_acc = q[0], k[0], v[0], out_acc[0], lse_acc[0]
        kw = {"into": (out_acc, lse_acc)} if fresh else {"accumulate_into": (out_acc, lse_acc)}
        fused(q, k, v, scale, tuple(window), causal, cu_q, cu_k, **kw)
        return
    if packed:
        out, lse = K.fwd_varlen(q[0], k[0], v[0], scale, tuple(window), cu_q, cu_k, None, None, causal)
        out, lse = out.unsqueeze(0), lse.unsqueeze(0)
    else:
        out, lse = K.fwd(q, k, v, scale, tuple(window), causal)
    if fresh:
        out_acc.copy_(out)
        lse_acc.copy_(lse)
    else:
        K.merge(out_acc, lse_acc, out, lse)


def _bwd_into(K, q, k, v, o, lse, do, dq, dk, dv, scale, window, causal, cu_q, cu_k, acc_dq, acc_dkv):
    """One block's gradients into ``dq, dk, dv`` (4-d views), written or added."""
    packed = cu_q is not None
    fused = getattr(K, "bwd_fused", None)
    if fused is not None:
        if packed:
            q, k, v, o, lse, do, dq, dk, dv = (t[0] for t in (q, k, v, o, lse, do, dq, dk, dv))
        fused(q, k, v, o, lse, do, dq, dk, dv, scale, tuple(window), causal, cu_q, cu_k,
              dq_accumulate=acc_dq, dkv_accumulate=acc_dkv)
        return
    wide = dq.dtype != q.dtype or dk.dtype != k.dtype
    if not (wide or acc_dq or acc_dkv):
        tq, tk, tv = dq, dk, dv
    else:
        tq, tk, tv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    if packed:
        K.bwd_varlen(q[0], k[0], v[0], o[0], lse[0], do[0], tq[0], tk[0], tv[0], scale,
                     tuple(window), cu_q, cu_k, None, None, causal)
    else:
        K.bwd(q, k, v, o, lse, do, tq, tk, tv, scale, tuple(window), causal)
    if tq is not dq:
        for dst, src, acc in ((dq, tq, acc_dq), (dk, tk, acc_dkv), (dv, tv, acc_dkv)):
            if acc:
                dst += src
            else:
                dst.copy_(src)


def _one_call(sq: int, sk: int, window_size: Tuple[int, int], causal: bool) -> bool:
    """Does the bottom-right window rule over the whole block equal upstream's two-part rule?"""
    if sq <= sk or (not causal and tuple(window_size) == (-1, -1)):
        return True
    right = 0 if causal else window_size[1]
    return right < 0 or right >= sq - 1


def flash_attn_fwd_func(
    q: torch.Tensor,
    kv: torch.Tensor,
    softmax_scale: float,
    window_size: Tuple[int, int],
    causal: bool,
    global_attn_out: torch.Tensor,
    global_softmax_lse: torch.Tensor,
    *,
    kernels: Optional[SimpleNamespace] = None,
    fresh: bool = False,
) -> None:
    """Dense block forward merged into the accumulators (``ops/attn.py:12-60``)."""
    K = kernels or hip_kernels()
    sq, sk = q.shape[1], kv[0].shape[1]
    if _one_call(sq, sk, window_size, causal):
        _fwd_into(K, q, kv[0], kv[1], softmax_scale, window_size, causal, None, None,
                  global_attn_out, global_softmax_lse, fresh)
        return
    # leading rows: every key; last Sk rows: the window
    flash_attn_fwd_func(q[:, :-sk], kv, softmax_scale, (-1, -1), False,
                        global_attn_out[:, :-sk], global_softmax_lse[:, :, :-sk], kernels=K,
                        fresh=fresh)
    flash_attn_fwd_func(q[:, -sk:], kv, softmax_scale, window_size, False,
                        global_attn_out[:, -sk:], global_softmax_lse[:, :, -sk:], kernels=K,
                        fresh=fresh)


def flash_attn_bwd_func(
    q: torch.Tensor,
    kv: torch.Tensor,
    o: torch.Tensor,
    softmax_lse: torch.Tensor,
    do: torch.Tensor,
    dq: torch.Tensor,
    dkv: torch.Tensor,
    softmax_scale: float,
    window_size: Tuple[int, int],
    causal: bool,
    *,
    kernels: Optional[SimpleNamespace] = None,
    accumulate_dq: bool = False,
    accumulate_dkv: bool = False,
) -> None:
    """Dense block backward into ``dq`` / ``dkv`` (``ops/attn.py:63-126``).  Sliced
    ``softmax_lse`` views are passed as they are (the kernels take strides; upstream clones
    them, ``:99-101``)."""
    K = kernels or hip_kernels()
    sq, sk = q.shape[1], kv[0].shape[1]
    if _one_call(sq, sk, window_size, causal):
        _bwd_into(K, q, kv[0], kv[1], o, softmax_lse, do, dq, dkv[0], dkv[1], softmax_scale,
                  window_size, causal, None, None, accumulate_dq, accumulate_dkv)
        return
    # two parts; dkv of the two summed in fp32 and rounded once, as upstream does (:93-126)
    parts = torch.zeros((2,) + tuple(kv[0].shape), dtype=torch.float32, device=q.device)
    flash_attn_bwd_func(q[:, :-sk], kv, o[:, :-sk], softmax_lse[:, :, :-sk], do[:, :-sk],
                        dq[:, :-sk], parts, softmax_scale, (-1, -1), causal, kernels=K,
                        accumulate_dq=accumulate_dq, accumulate_dkv=True)
    flash_attn_bwd_func(q[:, -sk:], kv, o[:, -sk:], softmax_lse[:, :, -sk:], do[:, -sk:],
                        dq[:, -sk:], parts, softmax_scale, window_size, causal, kernels=K,
                        accumulate_dq=accumulate_dq, accumulate_dkv=True)
    if accumulate_dkv:
        dkv += parts.to(kv[0].dtype)  # (the 16-bit block gradient, then the accumulator's sum)
    else:
        dkv.copy_(parts)


def flash_attn_varlen_fwd_func(
    q: torch.Tensor,
    kv: torch.Tensor,
    softmax_scale: float,
    window_size: Tuple[int, int],
    cu_seqlens_q: torch.Tensor,
    cu_seqlens_k: torch.Tensor,
    max_seqlen_q,
    max_seqlen_k,
    causal: bool,
    global_attn_out: torch.Tensor,
    global_softmax_lse: torch.Tensor,
    *,
    kernels: Optional[SimpleNamespace] = None,
    fresh: bool = False,
) -> None:
    """Packed block forward (batch dimension of size one around the pack, as upstream keeps
    it) merged into the accumulators (``ops/attn.py:129-160``).  ``max_seqlen_*`` are accepted
    for the signature and not needed."""
    K = kernels or hip_kernels()
    _fwd_into(K, q, kv[0], kv[1], softmax_scale, window_size, causal, cu_seqlens_q, cu_seqlens_k,
              global_attn_out, global_softmax_lse, fresh)


def flash_attn_varlen_bwd_func(
    q: torch.Tensor,
    kv: torch.Tensor,
    o: torch.Tensor,
    softmax_lse: torch.Tensor,
    do: torch.Tensor,
    dq: torch.Tensor,
    dkv: torch.Tensor,
    cu_seqlens_q: torch.Tensor,
    cu_seqlens_k: torch.Tensor,
    max_seqlen_q,
    max_seqlen_k,
    softmax_scale: float,
    window_size: Tuple[int, int],
    causal: bool,
    *,
    kernels: Optional[SimpleNamespace] = None,
    accumulate_dq: bool = False,
    accumulate_dkv: bool = False,
) -> None:
    """Packed block backward into ``dq`` / ``dkv`` (``ops/attn.py:163-196``)."""
    K = kernels or hip_kernels()
    _bwd_into(K, q, kv[0], kv[1], o, softmax_lse, do, dq, dkv[0], dkv[1], softmax_scale,
              window_size, causal, cu_seqlens_q, cu_seqlens_k, accumulate_dq, accumulate_dkv)
