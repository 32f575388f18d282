"""In-place LSE merge of two attention partials on the HIP kernel.

Same name, argument order and in-place contract as ``merge_attn_out`` of the
upstream package (``ring_swa/ops/merge.py:150-208``).
"""
from __future__ import annotations

import torch

from .. import _lib


def merge_attn_out(
    attn_out: torch.Tensor,
    softmax_lse: torch.Tensor,
    new_attn_out: torch.Tensor,
    new_softmax_lse: torch.Tensor,
) -> None:
    """Merge ``(new_attn_out, new_softmax_lse)`` into ``(attn_out, softmax_lse)``.

    attn_out / new_attn_out: ``[batch, seq, heads, dim]`` (bf16, fp16 or fp32);
    softmax_lse / new_softmax_lse: ``[batch, heads, seq]`` (fp32 or fp64).  Views
    with arbitrary outer strides are accepted; the last dim of the outputs must
    be contiguous.  ``lse = -inf`` is the identity on either side.
    """
    assert attn_out.dim() == 4 and new_attn_out.shape == attn_out.shape, "attn_out shape mismatch"
    b, s, h, d = attn_out.shape
    assert softmax_lse.shape == (b, h, s), "softmax_lse must be [batch, heads, seq]"
    assert new_softmax_lse.shape == (b, h, s), "new_softmax_lse must be [batch, heads, seq]"
    dev = _lib.require_device(attn_out, softmax_lse, new_attn_out, new_softmax_lse)
    L = _lib.lib()
    with torch.cuda.device(dev):
        st = L.rswa_merge_attn_out(
            attn_out.data_ptr(), _lib.dtype_code(attn_out), _lib.i64x4(attn_out.stride()),
            softmax_lse.data_ptr(), _lib.dtype_code(softmax_lse), _lib.i64x3(softmax_lse.stride()),
            new_attn_out.data_ptr(), _lib.dtype_code(new_attn_out),
            _lib.i64x4(new_attn_out.stride()),
            new_softmax_lse.data_ptr(), _lib.dtype_code(new_softmax_lse),
            _lib.i64x3(new_softmax_lse.stride()),
            b, s, h, d, _lib.stream_ptr(dev),
        )
    _lib.check(st)


def stream_copy(dst: torch.Tensor, src: torch.Tensor) -> None:
    """``dst <- src`` (contiguous device tensors of the same byte size, a multiple of 16) with
    the library's plain streaming-copy kernel: the yardstick the benchmark reports beside the
    merge kernel's rate (what a kernel that only moves memory reaches on the same device)."""
    assert dst.is_contiguous() and src.is_contiguous()
    nbytes = src.numel() * src.element_size()
    assert nbytes == dst.numel() * dst.element_size() and nbytes % 16 == 0
    dev = _lib.require_device(dst, src)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().rswa_stream_copy(dst.data_ptr(), src.data_ptr(), nbytes,
                                               _lib.stream_ptr(dev)))
