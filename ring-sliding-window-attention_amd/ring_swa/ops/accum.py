"""Block operators of the ring loops: one attention block merged into running accumulators
(forward), one block's gradients into caller buffers (backward).

Names, positional order and in-place behaviour of the four operators of the upstream package
(``ring_swa/ops/attn.py:12-60, 63-126, 129-160, 163-196``), so a ring loop written against
them runs on this package unchanged:

* ``kv`` is the stacked pair ``[2, batch, seq, kv_heads, dim]``;
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
        )
    return _HIP


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
) -> None:
    """Dense block forward merged into the accumulators (``ops/attn.py:12-60``)."""
    K = kernels or hip_kernels()
    sq, sk = q.shape[1], kv.shape[2]
    if _one_call(sq, sk, window_size, causal):
        out, lse = K.fwd(q, kv[0], kv[1], softmax_scale, tuple(window_size), causal)
        K.merge(global_attn_out, global_softmax_lse, out, lse)
        return
    # leading rows: every key; last Sk rows: the window
    flash_attn_fwd_func(q[:, :-sk], kv, softmax_scale, (-1, -1), False,
                        global_attn_out[:, :-sk], global_softmax_lse[:, :, :-sk], kernels=K)
    flash_attn_fwd_func(q[:, -sk:], kv, softmax_scale, window_size, False,
                        global_attn_out[:, -sk:], global_softmax_lse[:, :, -sk:], kernels=K)


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
) -> None:
    """Dense block backward into ``dq`` / ``dkv`` (``ops/attn.py:63-126``).  Sliced
    ``softmax_lse`` views are passed as they are (the kernels take strides; upstream clones
    them, ``:99-101``)."""
    K = kernels or hip_kernels()
    sq, sk = q.shape[1], kv.shape[2]
    if _one_call(sq, sk, window_size, causal):
        K.bwd(q, kv[0], kv[1], o, softmax_lse, do, dq, dkv[0], dkv[1], softmax_scale,
              tuple(window_size), causal)
        return
    # two parts; dkv of the two summed in fp32 and rounded once, as upstream does (:93-126)
    first = torch.empty_like(dkv)
    flash_attn_bwd_func(q[:, :-sk], kv, o[:, :-sk], softmax_lse[:, :, :-sk], do[:, :-sk],
                        dq[:, :-sk], first, softmax_scale, (-1, -1), causal, kernels=K)
    flash_attn_bwd_func(q[:, -sk:], kv, o[:, -sk:], softmax_lse[:, :, -sk:], do[:, -sk:],
                        dq[:, -sk:], dkv, softmax_scale, window_size, causal, kernels=K)
    dkv.copy_((first.float() + dkv.float()).to(dkv.dtype))


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
) -> None:
    """Packed block forward (batch dimension of size one around the pack, as upstream keeps
    it) merged into the accumulators (``ops/attn.py:129-160``).  ``max_seqlen_*`` are accepted
    for the signature and not needed."""
    K = kernels or hip_kernels()
    out, lse = K.fwd_varlen(q.squeeze(0), kv[0].squeeze(0), kv[1].squeeze(0), softmax_scale,
                            tuple(window_size), cu_seqlens_q, cu_seqlens_k, max_seqlen_q,
                            max_seqlen_k, causal)
    K.merge(global_attn_out, global_softmax_lse, out.unsqueeze(0), lse.unsqueeze(0))


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
) -> None:
    """Packed block backward into ``dq`` / ``dkv`` (``ops/attn.py:163-196``)."""
    K = kernels or hip_kernels()
    K.bwd_varlen(q.squeeze(0), kv[0].squeeze(0), kv[1].squeeze(0), o.squeeze(0),
                 softmax_lse.squeeze(0), do.squeeze(0), dq.squeeze(0), dkv[0].squeeze(0),
                 dkv[1].squeeze(0), softmax_scale, tuple(window_size), cu_seqlens_q,
                 cu_seqlens_k, max_seqlen_q, max_seqlen_k, causal)
