"""CPU oracle for the single-GPU attention path of ring_swa.

TEST INFRASTRUCTURE ONLY.  Nothing under ``oracle/`` is part of the product:
only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline``
leg may import it, and there only as the checker / the reported CPU baseline.

Every function is a plain PyTorch (CPU, fp32 or fp64) restatement of what the
reference computes on this path.  Citations are relative to the upstream
repository root:

* masked softmax attention with bottom-right aligned ``(left, right)`` window
  and GQA head mapping ............ ``test/test_local_swa.py:35-95``
* the same with the sink column forced on ... ``test/test_local_slm.py:14-73``
* log-sum-exp merge of two partials .......... ``ring_swa/ops/merge.py:16-50``
  (softplus form) and ``:132-147`` (sigmoid form)
* backward from externally supplied ``(o, lse)`` — the contract of
  ``ring_swa/ops/wrap_flash.py:276-327`` as used by
  ``ring_swa/sliding_window/nonvarlen.py:242-253`` and
  ``ring_swa/streaming_llm/naive.py:53-83``
* integer geometry of one ring rank's share ..
  ``ring_swa/sliding_window/nonvarlen.py:46-150`` and
  ``ring_swa/sliding_window/varlen.py:56-172``
* sink / window split of streaming-LLM ...... ``ring_swa/streaming_llm/naive.py:21-39,101-128``

Pinning status (see tests/test_oracle_pins.py): every function below is pinned
by a library routine, a closed form, a brute-force loop or ``gradcheck``; none
is "parity unpinned".  The third-party kernels the reference calls on this
path (flash-attn >= 2.5.8, not vendored, no lock file) cannot run here; their
published semantics (bottom-right aligned local window, natural-log LSE) are
what :func:`window_allowed` restates.
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import torch

NEG_INF = float("-inf")


# --------------------------------------------------------------------------
# masks
# --------------------------------------------------------------------------
def window_allowed(
    sq: int,
    sk: int,
    window: Tuple[int, int] = (-1, -1),
    causal: bool = False,
    n_sink: int = 0,
    device=None,
    shift: Optional[int] = None,
) -> torch.Tensor:
    """Boolean ``[sq, sk]`` matrix, True where query row i may see key j.

    ``shift`` (default ``sk - sq``): the key that query row 0 is aligned with; an explicit
    value moves the diagonal of the window rule (the out-of-window sink partial of the split
    streaming path uses ``-(window + 1)``).

    Bottom-right alignment: the last query row is aligned with the last key
    (``test/test_local_swa.py:63-85``).  ``causal`` forces the right extent to 0
    (flash-attn convention used at ``ring_swa/sliding_window/nonvarlen.py:379-386``).
    ``n_sink`` additionally allows keys ``j < n_sink`` that are not in the
    future of the query (``test/test_local_slm.py:58-63`` for one sink).
    """
    wl, wr = window
    if causal:
        wr = 0
    i = torch.arange(sq, device=device).unsqueeze(1)
    j = torch.arange(sk, device=device).unsqueeze(0)
    rel = j - i - ((sk - sq) if shift is None else shift)
    ok = torch.ones(sq, sk, dtype=torch.bool, device=device)
    if wl >= 0:
        ok &= rel >= -wl
    if wr >= 0:
        ok &= rel <= wr
    if n_sink > 0:
        sink = (j < n_sink).expand(sq, sk).clone()
        if wr >= 0:
            sink &= rel <= wr
        ok |= sink
    return ok


def global_band_allowed(
    positions_q: torch.Tensor,
    positions_k: torch.Tensor,
    seq_id_q: torch.Tensor,
    seq_id_k: torch.Tensor,
    window_size: int,
    n_sink: int = 0,
    seq_start_k: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """The one formula every call of the path reduces to.

    Query at global position p of sequence s sees key at global position t of
    the same sequence iff ``0 <= p - t <= window_size``
    (``ring_swa/sliding_window/nonvarlen.py:376-377``: w + 1 keys incl. self) or,
    for streaming-LLM, ``t - start(s) < n_sink`` and ``t <= p``
    (``ring_swa/streaming_llm/naive.py:21-39``).
    """
    p = positions_q.unsqueeze(1)
    t = positions_k.unsqueeze(0)
    same = seq_id_q.unsqueeze(1) == seq_id_k.unsqueeze(0)
    d = p - t
    ok = same & (d >= 0) & (d <= window_size)
    if n_sink > 0:
        assert seq_start_k is not None
        ok |= same & (d >= 0) & ((t - seq_start_k.unsqueeze(0)) < n_sink)
    return ok


# --------------------------------------------------------------------------
# forward
# --------------------------------------------------------------------------
def _expand_kv(x: torch.Tensor, hq: int) -> torch.Tensor:
    hk = x.shape[-2]
    assert hq % hk == 0, "q heads must be a multiple of kv heads"
    if hq == hk:
        return x
    # q head h uses kv head h // (hq / hk)   (test/test_local_swa.py:43-49)
    return x.repeat_interleave(hq // hk, dim=-2)


def masked_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    allowed: torch.Tensor,
    softmax_scale: Optional[float] = None,
    compute_dtype: torch.dtype = torch.float32,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Softmax attention under an explicit boolean mask.

    q ``[B,Sq,Hq,D]``, k/v ``[B,Sk,Hkv,D]``, allowed ``[Sq,Sk]`` (or
    ``[B,Sq,Sk]``).  Returns ``out [B,Sq,Hq,D]`` and ``lse [B,Hq,Sq]`` in
    ``compute_dtype``; rows with no allowed key give ``out = 0, lse = -inf``
    (the merge identity, ``ring_swa/ops/merge.py:138-147`` with ``g_lse=-inf``).
    Differentiable; one head at a time so the score matrix stays small.
    """
    b, sq, hq, d = q.shape
    if softmax_scale is None:
        softmax_scale = d ** (-0.5)
    qf = q.to(compute_dtype)
    kf = _expand_kv(k.to(compute_dtype), hq)
    vf = _expand_kv(v.to(compute_dtype), hq)
    if allowed.dim() == 2:
        allowed = allowed.unsqueeze(0)
    empty = ~allowed.any(dim=-1)  # [B or 1, Sq]
    outs, lses = [], []
    for h in range(hq):
        s = torch.einsum("bid,bjd->bij", qf[:, :, h], kf[:, :, h]) * softmax_scale
        s = s.masked_fill(~allowed, NEG_INF)
        lse = torch.logsumexp(s, dim=-1)  # -inf on empty rows
        safe = torch.where(torch.isinf(lse), torch.zeros_like(lse), lse)
        p = torch.exp(s - safe.unsqueeze(-1))
        p = p.masked_fill(empty.unsqueeze(-1), 0.0)
        outs.append(torch.einsum("bij,bjd->bid", p, vf[:, :, h]))
        lses.append(lse)
    return torch.stack(outs, dim=2), torch.stack(lses, dim=1)


def window_attention(
    q, k, v, softmax_scale=None, window=(-1, -1), causal=False, n_sink=0,
    compute_dtype=torch.float32, shift=None,
):
    """Dense block with flash-attn window semantics -> ``(out, lse)``.

    Restates ``ring_swa/ops/wrap_flash.py:168-200`` (what it returns) through
    the closed form of ``test/test_local_swa.py:51-93``.
    """
    allowed = window_allowed(q.shape[1], k.shape[1], window, causal, n_sink, device=q.device,
                             shift=shift)
    return masked_attention(q, k, v, allowed, softmax_scale, compute_dtype)


def window_attention_varlen(
    q, k, v, cu_seqlens_q, cu_seqlens_k, softmax_scale=None, window=(-1, -1),
    causal=False, n_sink=0, compute_dtype=torch.float32,
):
    """Packed variant: q ``[T,Hq,D]``; returns ``out [T,Hq,D]``, ``lse [Hq,T]``.

    Restates ``ring_swa/ops/wrap_flash.py:203-273``: each packed sequence is an
    independent dense block.
    """
    cq = [int(x) for x in cu_seqlens_q]
    ck = [int(x) for x in cu_seqlens_k]
    assert len(cq) == len(ck)
    outs, lses = [], []
    for b in range(len(cq) - 1):
        qs = q[cq[b]:cq[b + 1]].unsqueeze(0)
        ks = k[ck[b]:ck[b + 1]].unsqueeze(0)
        vs = v[ck[b]:ck[b + 1]].unsqueeze(0)
        if qs.shape[1] == 0:
            continue
        o, l = window_attention(qs, ks, vs, softmax_scale, window, causal, n_sink, compute_dtype)
        outs.append(o[0])
        lses.append(l[0])
    return torch.cat(outs, dim=0), torch.cat(lses, dim=1)


# --------------------------------------------------------------------------
# the four public functions, single-GPU semantics
# --------------------------------------------------------------------------
def sliding_window_attn(q, k, v, window_size, softmax_scale=None, compute_dtype=torch.float32):
    """``ring_sliding_window_attn(cp_group=None)``: ``ring_swa/sliding_window/nonvarlen.py:378-386``."""
    return window_attention(q, k, v, softmax_scale, (window_size, 0), True, 0, compute_dtype)


def sliding_window_attn_varlen(q, k, v, window_size, cu_seqlens, softmax_scale=None,
                               compute_dtype=torch.float32):
    """``ring_sliding_window_attn_varlen(cp_group=None)``: ``ring_swa/sliding_window/varlen.py:404-417``."""
    return window_attention_varlen(q, k, v, cu_seqlens, cu_seqlens, softmax_scale,
                                   (window_size, 0), True, 0, compute_dtype)


def streaming_llm_attn(q, k, v, window_size, softmax_scale=None, n_sink=1,
                       compute_dtype=torch.float32):
    """``ring_streaming_llm_attn(cp_group=None)``.

    Closed form of ``test/test_local_slm.py:34-71`` (band OR sink column).  The
    reference composes it as window-over-tokens-1.. plus one sink key merged by
    LSE (``ring_swa/streaming_llm/naive.py:21-39``); both give the same key set
    because key 0 is in the band exactly when ``p <= window_size``.
    """
    return window_attention(q, k, v, softmax_scale, (window_size, 0), True, n_sink, compute_dtype)


def streaming_llm_attn_varlen(q, k, v, window_size, cu_seqlens, softmax_scale=None, n_sink=1,
                              compute_dtype=torch.float32):
    """``ring_streaming_llm_attn_varlen(cp_group=None)`` with per-sequence sinks.

    The reference's forward takes the sink key/value from the first token of the
    whole pack (``ring_swa/streaming_llm/naive.py:116-117``) and requires all
    sequences to start with the same token (README precondition); under that
    precondition the two agree.
    """
    return window_attention_varlen(q, k, v, cu_seqlens, cu_seqlens, softmax_scale,
                                   (window_size, 0), True, n_sink, compute_dtype)


def streaming_llm_split_reference(q, k, v, window_size, softmax_scale=None,
                                  compute_dtype=torch.float32):
    """The reference's own composition, step by step, for one sink.

    ``ring_swa/streaming_llm/naive.py:21-39``: window attention over tokens 1..,
    full attention of every query to key 0, front-pad ``(0, -inf)``, LSE merge.
    Used to show the composition equals :func:`streaming_llm_attn`.
    """
    o_w, l_w = window_attention(q[:, 1:], k[:, 1:], v[:, 1:], softmax_scale,
                                (window_size, 0), True, 0, compute_dtype)
    o_s, l_s = window_attention(q, k[:, :1], v[:, :1], softmax_scale, (-1, -1), False, 0,
                                compute_dtype)
    o = torch.nn.functional.pad(o_w, (0, 0, 0, 0, 1, 0), value=0.0)
    l = torch.nn.functional.pad(l_w, (1, 0), value=NEG_INF)
    return merge(o, l, o_s, l_s)


# --------------------------------------------------------------------------
# merge
# --------------------------------------------------------------------------
def merge(o, lse, o_new, lse_new):
    """Out-of-place LSE merge, sigmoid form (``ring_swa/ops/merge.py:137-147``).

    ``o [B,S,H,D]``, ``lse [B,H,S]``.  Returns ``(o_merged, lse_merged)`` in the
    dtype of ``o`` / ``lse``; arithmetic in fp32 as the Triton kernel does
    (``:134-135``) unless ``lse`` is fp64 *and* ``o`` is fp64.  ``-inf`` on either
    side is the identity; both ``-inf`` gives ``(0, -inf)`` (the reference yields NaN there).
    """
    cd = torch.float64 if (lse.dtype == torch.float64 and o.dtype == torch.float64) else torch.float32
    a = lse.to(cd)
    b = lse_new.to(cd)
    both_empty = torch.isinf(a) & torch.isinf(b) & (a < 0) & (b < 0)
    diff = torch.where(both_empty, torch.zeros_like(a), b - a)
    w_old = torch.sigmoid(-diff).masked_fill(both_empty, 0.0)
    w_new = torch.sigmoid(diff).masked_fill(both_empty, 0.0)
    w_old_b = w_old.movedim(1, 2).unsqueeze(-1)
    w_new_b = w_new.movedim(1, 2).unsqueeze(-1)
    o_m = o.to(cd) * w_old_b + o_new.to(cd) * w_new_b
    m = torch.maximum(a, b)
    l_m = m + torch.log1p(torch.exp(-diff.abs()))
    l_m = torch.where(both_empty, torch.full_like(l_m, NEG_INF), l_m)
    return o_m.to(o.dtype), l_m.to(lse.dtype)


def merge_softplus(o, lse, o_new, lse_new):
    """The torch fallback's softplus form (``ring_swa/ops/merge.py:30-50``), out of place."""
    a = lse
    b = lse_new.to(lse.dtype)
    diff = b - a
    scale = torch.exp(-torch.nn.functional.softplus(diff)).movedim(1, 2).unsqueeze(-1)
    new_scale = torch.exp(-torch.nn.functional.softplus(-diff)).movedim(1, 2).unsqueeze(-1)
    o_m = o * scale + o_new * new_scale
    l_m = torch.maximum(a, b) + torch.log1p(torch.exp(-diff.abs()))
    return o_m.to(o.dtype), l_m


# --------------------------------------------------------------------------
# backward from supplied statistics
# --------------------------------------------------------------------------
def attention_bwd_from_stats(
    q, k, v, o, lse, do, allowed, softmax_scale=None, compute_dtype=torch.float32
):
    """Gradients of one block given the *final* ``(o, lse)`` of the row.

    Contract of ``ring_swa/ops/wrap_flash.py:276-327`` as the ring uses it
    (``ring_swa/sliding_window/nonvarlen.py:242-253``): ``P = exp(scale*q.k - lse)``
    restricted to ``allowed``, ``delta = rowsum(do*o)``, ``dV = P^T dO``,
    ``dS = P * (dO V^T - delta)``, ``dQ = scale * dS K``, ``dK = scale * dS^T Q``;
    dK/dV summed over the q heads sharing a kv head.  Returns ``(dq, dk, dv)`` in
    ``compute_dtype``.
    """
    b, sq, hq, d = q.shape
    hk = k.shape[2]
    g = hq // hk
    if softmax_scale is None:
        softmax_scale = d ** (-0.5)
    qf, kf, vf = (t.to(compute_dtype) for t in (q, k, v))
    of, dof, lf = o.to(compute_dtype), do.to(compute_dtype), lse.to(compute_dtype)
    if allowed.dim() == 2:
        allowed = allowed.unsqueeze(0)
    dq = torch.zeros_like(qf)
    dk = torch.zeros_like(kf)
    dv = torch.zeros_like(vf)
    for h in range(hq):
        hh = h // g
        s = torch.einsum("bid,bjd->bij", qf[:, :, h], kf[:, :, hh]) * softmax_scale
        l = lf[:, h]
        safe = torch.where(torch.isinf(l), torch.zeros_like(l), l)
        p = torch.exp(s - safe.unsqueeze(-1)).masked_fill(~allowed, 0.0)
        p = p.masked_fill(torch.isinf(l).unsqueeze(-1), 0.0)
        delta = (dof[:, :, h] * of[:, :, h]).sum(-1)
        dp = torch.einsum("bid,bjd->bij", dof[:, :, h], vf[:, :, hh])
        ds = p * (dp - delta.unsqueeze(-1))
        dv[:, :, hh] += torch.einsum("bij,bid->bjd", p, dof[:, :, h])
        dq[:, :, h] = softmax_scale * torch.einsum("bij,bjd->bid", ds, kf[:, :, hh])
        dk[:, :, hh] += softmax_scale * torch.einsum("bij,bid->bjd", ds, qf[:, :, h])
    return dq, dk, dv


def attention_fwd_bwd(fn, q, k, v, do, *args, **kwargs):
    """Run ``fn(q,k,v,*args) -> (out, lse)`` with autograd and return ``(out, lse, dq, dk, dv)``."""
    q = q.detach().clone().requires_grad_()
    k = k.detach().clone().requires_grad_()
    v = v.detach().clone().requires_grad_()
    out, lse = fn(q, k, v, *args, **kwargs)
    out.backward(do.to(out.dtype))
    return out.detach(), lse.detach(), q.grad, k.grad, v.grad


# --------------------------------------------------------------------------
# geometry of one ring rank's share (integers only)
# --------------------------------------------------------------------------
def ring_steps_nonvarlen(seq_len: int, window_size: int, cp_size: int, rank: int):
    """Blocks one rank computes, as ``(step, q_slice, kv_slice, window, causal)``.

    Follows ``ring_swa/sliding_window/nonvarlen.py:46-150``: step i uses the KV
    chunk of rank ``rank - i``; slices are Python ``slice`` objects on the local
    sequence axis; wrap-around steps (``rank - i < 0``) are skipped (``:97``).
    """
    steps = []
    times = min(math.ceil(window_size / seq_len), cp_size - 1)
    full = slice(0, seq_len)
    for i in range(times + 1):
        if rank - i < 0:
            continue
        if i == 0:
            steps.append((i, full, full, (window_size, 0), True))
        elif (i + 1) * seq_len <= window_size + 1:
            steps.append((i, full, full, (-1, -1), False))
        elif (i + 1) * seq_len > window_size + 1 > i * seq_len:
            steps.append((i, full, full, (window_size % seq_len, seq_len), False))
        elif i * seq_len > window_size > (i - 1) * seq_len:
            vl = window_size % seq_len
            steps.append((i, slice(0, vl), slice(seq_len - vl, seq_len), (0, seq_len), False))
        else:
            raise ValueError(f"invalid step {i}")
    return steps


def ring_steps_varlen(cu_seqlens: Sequence[int], seq_len: int, window_size: int,
                      cp_size: int, rank: int):
    """Varlen twin, following ``ring_swa/sliding_window/varlen.py:56-172``.

    Returns ``(local_cu_seqlens, steps)``; the diagonal step carries
    ``local_cu_seqlens`` and off-diagonal steps are dense rectangles on the
    rank's first (straddling) sequence.
    """
    cu = [int(x) for x in cu_seqlens]
    start = rank * seq_len
    end = start + seq_len
    first = next(i for i, c in enumerate(cu) if c > start)
    last = next(i for i, c in enumerate(cu) if c >= end)
    local_cu = [0] + [c - start for c in cu[first:last]] + [seq_len]
    first_q_len = local_cu[1]
    first_kv_len = start - cu[first - 1]
    times = min(math.ceil(window_size / seq_len), cp_size - 1)
    steps = [(0, slice(0, seq_len), slice(0, seq_len), (window_size, 0), True)]
    for i in range(1, times + 1):
        if rank - i < 0:
            continue
        if min(first_kv_len, window_size) > (i - 1) * seq_len:
            vk = min(first_kv_len - (i - 1) * seq_len, seq_len)
            vq = first_q_len
            vw = min(window_size - (i - 1) * seq_len, seq_len * 2)
            vq = min(vq, vw)
            vk = min(vk, vw)
            steps.append((i, slice(0, vq), slice(seq_len - vk, seq_len), (vw - vq, seq_len), False))
    return local_cu, steps


# --------------------------------------------------------------------------
# work counters (the FLOP model of the headline metric: 4 D per pair forward, 10 D backward)
# --------------------------------------------------------------------------
def band_pairs(length: int, window_size: int) -> int:
    """Unmasked (query,key) pairs of one sequence: closed form ``P(L,w)``."""
    if length <= window_size + 1:
        return length * (length + 1) // 2
    return (window_size + 1) * length - window_size * (window_size + 1) // 2


def sink_extra_pairs(length: int, window_size: int, n_sink: int) -> int:
    """Out-of-window sink pairs of one sequence."""
    m = length - 1 - window_size
    if m <= 0 or n_sink <= 0:
        return 0
    if m <= n_sink:
        return m * (m + 1) // 2
    return n_sink * (n_sink + 1) // 2 + n_sink * (m - n_sink)


def attention_flops(pairs: int, head_dim: int, n_q_heads: int, batch: int = 1):
    """``(fwd, bwd, total)`` FLOPs: 4, 10 and 14 times ``D * pairs * Hq * B``."""
    unit = head_dim * pairs * n_q_heads * batch
    return 4 * unit, 10 * unit, 14 * unit
