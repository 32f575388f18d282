"""Kernel-level attention operators: one masked block, forward or backward.

These take the place of the flash-attn wrappers of the upstream package
(``ring_swa/ops/wrap_flash.py:168-429``) and keep their names, positional
argument order and conventions:

* ``window_size = (left, right)``, ``-1`` = unbounded, bottom-right aligned;
  ``causal=True`` forces ``right = 0``;
* forward returns ``(out, softmax_lse)`` with ``softmax_lse`` fp32
  ``[batch, heads, seq]`` (dense) or ``[heads, total]`` (packed);
* backward writes into the caller's ``dq, dk, dv`` and uses the caller's
  ``o`` / ``softmax_lse`` (which may be merged statistics).

Additions (keyword-only): ``num_sink`` (attention-sink keys at the head of each
sequence, visible regardless of the left window bound) and, on ``attn_fwd`` /
``attn_bwd``, ``mask_shift`` (explicit diagonal offset replacing the bottom-right
``len_k - len_q``).  Rows without any
visible key produce ``out = 0``, ``lse = -inf`` (the merge identity).
"""
from __future__ import annotations

import os

from typing import Optional, Tuple

import torch

from .. import _lib


def _check_qkv(q, k, v, packed: bool):
    nd = 3 if packed else 4
    assert q.dim() == nd and k.dim() == nd and v.dim() == nd, (
        f"expected {nd}-d q/k/v, got {q.dim()}, {k.dim()}, {v.dim()}"
    )
    assert k.shape == v.shape, "k and v must have the same shape"
    assert q.shape[-1] == k.shape[-1], "head_dim mismatch"
    assert q.dtype == k.dtype == v.dtype, "q, k, v must share a dtype"
    assert q.shape[-2] % k.shape[-2] == 0, (
        "Number of query heads must be divisible by number of key/value heads"
    )
    if not packed:
        assert q.shape[0] == k.shape[0], "batch mismatch"
    for t in (q, k, v):
        assert t.stride(-1) == 1, "last dimension must be contiguous"


def _strides3(t: torch.Tensor, packed: bool):
    if packed:
        return (0, t.stride(0), t.stride(1))
    return (t.stride(0), t.stride(1), t.stride(2))


def _lse_strides(lse: torch.Tensor, packed: bool):
    if packed:
        return (0, lse.stride(0), lse.stride(1))
    return (lse.stride(0), lse.stride(1), lse.stride(2))


def _same_strides(a, b) -> bool:
    """Do ``a`` and ``b`` step alike through memory?  (A stride over one element is never used.)"""
    return all(a.stride(d) == b.stride(d) for d in range(a.dim())
               if a.shape[d] > 1 and b.shape[d] > 1)


def _second_range(p, k, v, second, packed):
    """Keys in two row ranges: ``(k, v)`` first, then ``second = (k2, v2)`` (dense, same batch,
    heads, head_dim and strides; ``k.shape[1]`` a multiple of 256)."""
    k2, v2 = second[0], second[1]
    assert not packed, "two key ranges in dense mode only"
    for a, b in ((k, k2), (v, v2)):
        assert b.dim() == 4 and b.dtype == a.dtype and b.shape[0] == a.shape[0] and \
            b.shape[2:] == a.shape[2:], "the second key range must match the first but for its rows"
        assert _same_strides(a, b), "the two key ranges must have the same strides"
    assert k2.shape == v2.shape and k2.shape[1] > 0
    assert k.shape[1] > 0 and k.shape[1] % 256 == 0, (
        "the first key range must hold a positive multiple of 256 rows")
    p.seqlen_k = k.shape[1] + k2.shape[1]
    p.seg_rows = k.shape[1]
    p.k2, p.v2 = k2.data_ptr(), v2.data_ptr()


def _params(q, k, v, softmax_scale, window_size, causal, cu_q, cu_k, num_sink,
            mask_shift=None, second=None) -> "_lib.AttnParams":
    packed = cu_q is not None
    p = _lib.AttnParams()
    p.dtype = _lib.dtype_code(q)
    p.head_dim = q.shape[-1]
    p.heads_q = q.shape[-2]
    p.heads_kv = k.shape[-2]
    if packed:
        assert cu_k is not None, "cu_seqlens_k is required with cu_seqlens_q"
        for cu in (cu_q, cu_k):
            assert cu.dtype == torch.int32 and cu.dim() == 1 and cu.is_contiguous(), (
                "cu_seqlens must be a contiguous 1-d int32 tensor"
            )
            assert cu.device == q.device, "cu_seqlens must live on the tensors' device"
        assert cu_q.numel() == cu_k.numel() and cu_q.numel() >= 2
        p.batch = cu_q.numel() - 1
        p.total_q, p.total_k = q.shape[0], k.shape[0]
        # only upper bounds are needed, so no device->host read of the lengths
        p.seqlen_q, p.seqlen_k = q.shape[0], k.shape[0]
        p.cu_seqlens_q, p.cu_seqlens_k = cu_q.data_ptr(), cu_k.data_ptr()
    else:
        p.batch = q.shape[0]
        p.seqlen_q, p.seqlen_k = q.shape[1], k.shape[1]
        p.total_q = p.total_k = 0
        p.cu_seqlens_q = p.cu_seqlens_k = None
    p.softmax_scale = float(softmax_scale)
    p.window_left, p.window_right = int(window_size[0]), int(window_size[1])
    p.causal = 1 if causal else 0
    p.num_sink = int(num_sink)
    p.shift_explicit = 0 if mask_shift is None else 1
    p.shift = 0 if mask_shift is None else int(mask_shift)
    p.q, p.k, p.v = q.data_ptr(), k.data_ptr(), v.data_ptr()
    p.q_stride = _lib.i64x3(_strides3(q, packed))
    p.k_stride = _lib.i64x3(_strides3(k, packed))
    p.v_stride = _lib.i64x3(_strides3(v, packed))
    # RSWA_ADDRESSING=far: the kernels that base every tile fetch at the tile's own first row
    # (picked by the library itself once a sequence spans 2 GiB) whatever the sizes
    p.addressing = 1 if os.environ.get("RSWA_ADDRESSING", "") == "far" else 0
    if second is not None:
        _second_range(p, k, v, second, packed)
    return p


def attn_fwd(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    softmax_scale: Optional[float],
    window_size: Tuple[int, int] = (-1, -1),
    causal: bool = False,
    cu_seqlens_q: Optional[torch.Tensor] = None,
    cu_seqlens_k: Optional[torch.Tensor] = None,
    *,
    num_sink: int = 0,
    mask_shift: Optional[int] = None,
    accumulate_into: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
    second: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
    into: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Masked attention forward on the HIP kernel; returns ``(out, lse)``.

    ``second=(k2, v2)``: the keys are the rows of ``k`` followed by the rows of ``k2`` (dense
    mode; same strides; ``k.shape[1]`` a multiple of 256), taken where they lie -- a ring
    rank's tail of the previous chunk and its own chunk in one pass, without a concatenation.

    ``accumulate_into=(out, lse)``: running partial results of these rows (``out`` in q's
    dtype, ``lse`` fp32, views allowed) that this block is merged into in place, in the
    kernel's epilogue -- the same bits as a forward into temporaries followed by
    ``merge_attn_out``, without the temporaries and the second pass.  The pair may also be the
    ring loops' accumulators, ``out`` fp32 and ``lse`` fp64
    (``ring_swa/sliding_window/nonvarlen.py:53-59``).

    ``into=(out, lse)``: write the block's result into these buffers instead of fresh ones (same
    two type pairs; as fp32 the values are the block's 16-bit output, exactly) -- how a ring loop
    starts its accumulators without zero-filling them first."""
    packed = cu_seqlens_q is not None
    _check_qkv(q, k, v, packed)
    assert second is None or k.numel() > 0, "two key ranges: the first must not be empty"
    dev = _lib.require_device(q, k, v)
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** (-0.5)
    lse_shape = (q.shape[1], q.shape[0]) if packed else (q.shape[0], q.shape[2], q.shape[1])
    wide = False
    assert accumulate_into is None or into is None
    if accumulate_into is not None or into is not None:
        out, lse = accumulate_into if accumulate_into is not None else into
        wide = out.dtype == torch.float32
        assert out.shape == q.shape and out.stride(-1) == 1 and tuple(lse.shape) == lse_shape, (
            "out must have q's shape, lse [batch, heads, seq] ([heads, tokens] when packed)"
        )
        assert (out.dtype, lse.dtype) in ((q.dtype, torch.float32), (torch.float32, torch.float64)), (
            "out / lse must be q's dtype / fp32, or the ring accumulators' fp32 / fp64"
        )
        _lib.require_device(out, lse)
        if accumulate_into is not None and (q.numel() == 0 or k.numel() == 0):
            return out, lse  # an empty block is the identity of the merge
        if into is not None and (q.numel() == 0 or k.numel() == 0):
            out.zero_()
            lse.fill_(float("-inf"))
            return out, lse
    else:
        out = torch.empty(q.shape, dtype=q.dtype, device=dev)
        lse = torch.empty(lse_shape, dtype=torch.float32, device=dev)
        if q.numel() == 0:
            return out, lse
        if k.numel() == 0:
            # no keys at all: every row is empty (out = 0, lse = -inf), as attn_bwd assumes
            out.zero_()
            lse.fill_(float("-inf"))
            return out, lse
    p = _params(q, k, v, softmax_scale, window_size, causal, cu_seqlens_q, cu_seqlens_k, num_sink,
                mask_shift, second)
    p.out = out.data_ptr()
    p.out_stride = _lib.i64x3(_strides3(out, packed))
    p.lse = lse.data_ptr()
    p.lse_stride = _lib.i64x3(_lse_strides(lse, packed))
    p.out_accumulate = 0 if accumulate_into is None else 1
    p.wide = _lib.WIDE_OUT if wide else 0
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().rswa_attn_fwd(p, _lib.stream_ptr(dev)))
    return out, lse


def attn_bwd(
    q, k, v, o, softmax_lse, do, dq, dk, dv,
    softmax_scale: Optional[float],
    window_size: Tuple[int, int] = (-1, -1),
    causal: bool = False,
    cu_seqlens_q: Optional[torch.Tensor] = None,
    cu_seqlens_k: Optional[torch.Tensor] = None,
    *,
    num_sink: int = 0,
    mask_shift: Optional[int] = None,
    workspace: Optional[torch.Tensor] = None,
    phases: int = 7,
    dq_accumulate: bool = False,
    static_workspace: bool = False,
    second: Optional[Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]] = None,
    handoff=None,
    dkv_accumulate: bool = False,
) -> None:
    """Masked attention backward; overwrites ``dq, dk, dv`` (views are fine).

    ``second=(k2, v2, dk2, dv2)``: keys in two row ranges as in ``attn_fwd``; the gradients of
    the second range's rows go to ``dk2, dv2`` (shapes and strides of ``k2, v2``).

    ``workspace`` (uint8, at least ``bwd_workspace_bytes(q, k, ...)``) may be supplied to avoid the
    per-call scratch allocation, and must be when the phases of one backward are spread
    over several calls; ``phases`` is the bit mask of ``rswa_attn_bwd_phases`` (1 prep,
    2 dk/dv kernel, 4 dq kernel).  ``dq_accumulate`` adds this call's dQ to the values
    already in ``dq`` (fp32 add of the two 16-bit values, one rounding).
    ``static_workspace=True`` runs the whole backward on the library's built-in statistics
    buffer (``rswa_attn_bwd_static``): no device memory is allocated by the call; sizes
    beyond the buffer raise ``NotImplementedError`` and overlapping calls on one GPU race.

    ``dq``, and ``dk`` / ``dv`` together, may also be fp32 -- the ring loops' gradient accumulators
    (``ring_swa/sliding_window/nonvarlen.py:203-206``): the block's 16-bit gradients are then
    written as fp32, or with ``dq_accumulate`` / ``dkv_accumulate`` (fp32 ``dk`` / ``dv`` only)
    added to what the buffers hold, the sums of ``:318-321`` without their elementwise passes.

    ``handoff``: dS hand-off (``ds_handoff`` of the ABI) -- the dK/dV kernel stores its 16-bit dS
    tiles in the workspace and dQ comes from a kernel that only multiplies them with K instead
    of recomputing S and dP.  ``None`` (default) takes it when the library accepts the shape and
    the tiles fit ``handoff_max_bytes()`` (0 unless the environment switches the route on: it is
    not faster at the sizes measured); ``True`` asks for it whatever its size (shapes the
    library does not accept still take the recomputing route, and so do small launches whose key
    tiles the dK/dV kernel splits over several blocks -- ``"force"`` prefers the hand-off to that
    split); ``False`` never.  With
    ``phases`` spread over several calls the same value must be passed to each, on the same
    workspace, and the dK/dV phase must run before the dQ phase.  A ``workspace`` the caller
    supplies without room for the dS tiles makes the automatic choice (``None``) recompute."""
    packed = cu_seqlens_q is not None
    _check_qkv(q, k, v, packed)
    assert second is None or k.numel() > 0, "two key ranges: the first must not be empty"
    dev = _lib.require_device(q, k, v, o, softmax_lse, do, dq, dk, dv)
    assert o.shape == q.shape and do.shape == q.shape and dq.shape == q.shape
    assert dk.shape == k.shape and dv.shape == v.shape
    assert o.dtype == q.dtype and do.dtype == q.dtype
    assert dq.dtype in (q.dtype, torch.float32) and dk.dtype in (q.dtype, torch.float32) and \
        dv.dtype == dk.dtype, "dq and dk / dv must have the dtype of q, or be fp32 accumulators"
    wide_dq, wide_dkv = dq.dtype == torch.float32, dk.dtype == torch.float32
    assert not dkv_accumulate or wide_dkv, "dkv_accumulate needs fp32 dk / dv"
    assert softmax_lse.dtype == torch.float32, "softmax_lse must be fp32"
    for t in (o, do, dq, dk, dv):
        assert t.stride(-1) == 1, "last dimension must be contiguous"
    if packed:
        assert softmax_lse.shape == (q.shape[1], q.shape[0])
    else:
        assert softmax_lse.shape == (q.shape[0], q.shape[2], q.shape[1])
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** (-0.5)
    if q.numel() == 0 or k.numel() == 0:
        # nothing to attend: the outputs of the requested phases are zero
        if (phases & 4) and not dq_accumulate:
            dq.zero_()
        if (phases & 2) and not dkv_accumulate:
            dk.zero_()
            dv.zero_()
        return
    p = _params(q, k, v, softmax_scale, window_size, causal, cu_seqlens_q, cu_seqlens_k, num_sink,
                mask_shift, second)
    if second is not None:
        dk2, dv2 = second[2], second[3]
        _lib.require_device(dk2, dv2)
        assert dk2.shape == second[0].shape and dv2.shape == second[1].shape
        assert dk2.dtype == dk.dtype and dv2.dtype == dk.dtype
        assert _same_strides(dk2, dk) and _same_strides(dv2, dv), (
            "dk2 / dv2 must have the strides of dk / dv"
        )
        p.dk2, p.dv2 = dk2.data_ptr(), dv2.data_ptr()
    p.dq_accumulate = int(bool(dq_accumulate))
    p.dkv_accumulate = int(bool(dkv_accumulate))
    p.wide = (_lib.WIDE_DQ if wide_dq else 0) | (_lib.WIDE_DKV if wide_dkv else 0)
    p.out = o.data_ptr()
    p.out_stride = _lib.i64x3(_strides3(o, packed))
    p.lse = softmax_lse.data_ptr()
    p.lse_stride = _lib.i64x3(_lse_strides(softmax_lse, packed))
    p.dout = do.data_ptr()
    p.dout_stride = _lib.i64x3(_strides3(do, packed))
    p.dq, p.dk, p.dv = dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
    p.dq_stride = _lib.i64x3(_strides3(dq, packed))
    p.dk_stride = _lib.i64x3(_strides3(dk, packed))
    p.dv_stride = _lib.i64x3(_strides3(dv, packed))
    L = _lib.lib()
    if static_workspace:
        assert phases == 7 and workspace is None, "the built-in buffer serves whole backward calls"
        with torch.cuda.device(dev):
            _lib.check(L.rswa_attn_bwd_static(p, _lib.stream_ptr(dev)))
        return
    _set_handoff(p, handoff)
    need = int(L.rswa_attn_bwd_workspace_bytes(p))
    if workspace is not None and handoff is None and p.ds_handoff and workspace.numel() < need:
        # a caller's workspace without room for the dS tiles: the automatic choice recomputes
        p.ds_handoff = 0
        need = int(L.rswa_attn_bwd_workspace_bytes(p))
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=dev)  # 512-B aligned by torch
    assert workspace.dtype == torch.uint8 and workspace.device == dev
    assert workspace.numel() >= need, (
        f"workspace of {workspace.numel()} bytes, {need} needed: size it with bwd_workspace_bytes "
        "and the mask / num_sink / handoff of this call"
    )
    p.workspace = workspace.data_ptr()
    p.workspace_bytes = workspace.numel()
    with torch.cuda.device(dev):
        _lib.check(L.rswa_attn_bwd_phases(p, _lib.stream_ptr(dev), int(phases)))


def bwd_static_init(device=None) -> None:
    """Resolve the address of the built-in statistics buffer of ``attn_bwd(static_workspace=True)``
    on ``device`` (default: the current one).  The first such backward on a device does it by
    itself; call this before capturing one into a HIP graph, where the look-up must not happen."""
    with torch.cuda.device(device):
        _lib.check(_lib.lib().rswa_attn_bwd_static_init())


def handoff_max_bytes() -> int:
    """Largest dS buffer ``attn_bwd(handoff=None)`` takes by itself.  0 unless the environment
    asks for the route (``RSWA_DS_HANDOFF=1``; then ``RSWA_DS_HANDOFF_MAX_BYTES`` or 8 GiB): measured
    on an MI355X the route is within +-5 % of the recomputing one at every size tried (faster
    at windows of a few hundred keys, slower at thousands: writing and reading 2 bytes per
    (query, key) pair costs what the saved matrix work gains), so it is not taken by default."""
    if os.environ.get("RSWA_DS_HANDOFF", "0") != "1":
        return 0
    return int(os.environ.get("RSWA_DS_HANDOFF_MAX_BYTES", 8 << 30))


def _set_handoff(p, handoff: Optional[bool]) -> bool:
    """Decide ``p.ds_handoff`` (see ``attn_bwd``); returns whether the library will take it."""
    L = _lib.lib()
    p.ds_handoff = 0
    if handoff is False:
        return False
    p.ds_handoff = 2 if handoff == "force" else 1
    if not L.rswa_attn_bwd_handoff_active(p):
        p.ds_handoff = 0
        return False
    if handoff is None:
        if handoff_max_bytes() == 0:
            p.ds_handoff = 0
            return False
        with_ds = int(L.rswa_attn_bwd_workspace_bytes(p))
        p.ds_handoff = 0
        if with_ds - int(L.rswa_attn_bwd_workspace_bytes(p)) > handoff_max_bytes():
            return False
        p.ds_handoff = 1
    return True


def bwd_workspace_bytes(q: torch.Tensor, k: torch.Tensor,
                        cu_seqlens_q: Optional[torch.Tensor] = None,
                        cu_seqlens_k: Optional[torch.Tensor] = None, *,
                        second_rows: int = 0,
                        window_size: Tuple[int, int] = (-1, -1), causal: bool = False,
                        num_sink: int = 0, handoff: Optional[bool] = False) -> int:
    """Scratch size of one backward over ``q`` against ``k`` (dense ``[B,S,H,D]`` or packed
    ``[T,H,D]``), as ``rswa_attn_bwd_workspace_bytes`` computes it: two fp32 values per
    (row, q head); the partial sums of the dK/dV kernel when the shape makes it deal the q
    heads of a GQA group to several blocks; the sums of the sink kernel with ``num_sink`` keys
    under a bounded window; the dS tiles with ``handoff`` (which depend on the window).  Pass the
    mask and ``handoff`` of the ``attn_bwd`` call the workspace is for."""
    p = _params(q, k, k, 1.0, window_size, causal, cu_seqlens_q, cu_seqlens_k, num_sink)
    p.seqlen_k += int(second_rows)  # keys in two row ranges: the rows of the second
    p.dout_stride = p.q_stride
    _set_handoff(p, handoff)
    return int(_lib.lib().rswa_attn_bwd_workspace_bytes(p))


def bwd_handoff_active(q: torch.Tensor, k: torch.Tensor,
                       cu_seqlens_q: Optional[torch.Tensor] = None,
                       cu_seqlens_k: Optional[torch.Tensor] = None, *,
                       second_rows: int = 0,
                       window_size: Tuple[int, int] = (-1, -1), causal: bool = False,
                       num_sink: int = 0, handoff: Optional[bool] = None) -> bool:
    """Would ``attn_bwd`` with these arguments take the dS hand-off route?"""
    p = _params(q, k, k, 1.0, window_size, causal, cu_seqlens_q, cu_seqlens_k, num_sink)
    p.seqlen_k += int(second_rows)
    p.dout_stride = p.q_stride
    return _set_handoff(p, handoff)


# ---- names of the upstream wrappers -----------------------------------------
def wrapped_flash_attn_fwd(q, k, v, softmax_scale, window_size, causal, *, num_sink=0,
                           mask_shift=None):
    """Dense forward, ``ring_swa/ops/wrap_flash.py:168``: returns ``(out, softmax_lse)``.
    ``mask_shift`` replaces the bottom-right alignment ``len_k - len_q`` of the window rule."""
    return attn_fwd(q, k, v, softmax_scale, window_size, causal, num_sink=num_sink,
                    mask_shift=mask_shift)


def wrapped_flash_attn_fwd_varlen(
    q, k, v, softmax_scale, window_size, cu_seqlens_q, cu_seqlens_k,
    max_seqlen_q=None, max_seqlen_k=None, causal=False, *, num_sink=0, mask_shift=None,
):
    """Packed forward, ``ring_swa/ops/wrap_flash.py:203``.  ``max_seqlen_*`` are
    accepted for signature compatibility and unused (no host sync is needed)."""
    return attn_fwd(q, k, v, softmax_scale, window_size, causal, cu_seqlens_q, cu_seqlens_k,
                    num_sink=num_sink, mask_shift=mask_shift)


def wrapped_flash_attn_bwd(
    q, k, v, o, softmax_lse, do, dq, dk, dv, softmax_scale, window_size, causal, *, num_sink=0,
    mask_shift=None,
):
    """Dense backward, ``ring_swa/ops/wrap_flash.py:276``; fills ``dq, dk, dv``."""
    attn_bwd(q, k, v, o, softmax_lse, do, dq, dk, dv, softmax_scale, window_size, causal,
             num_sink=num_sink, mask_shift=mask_shift)


def wrapped_flash_attn_bwd_varlen(
    q, k, v, o, softmax_lse, do, dq, dk, dv, softmax_scale, window_size,
    cu_seqlens_q, cu_seqlens_k, max_seqlen_q=None, max_seqlen_k=None, causal=False, *,
    num_sink=0, mask_shift=None,
):
    """Packed backward, ``ring_swa/ops/wrap_flash.py:330``; fills ``dq, dk, dv``."""
    attn_bwd(q, k, v, o, softmax_lse, do, dq, dk, dv, softmax_scale, window_size, causal,
             cu_seqlens_q, cu_seqlens_k, num_sink=num_sink, mask_shift=mask_shift)
