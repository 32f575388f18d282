"""ctypes binding of librswa.so (the C ABI declared in include/rswa.h).

The library is the only compute path: there is no fallback.  Loading fails
loudly when the shared object has not been built.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import (POINTER, Structure, c_char_p, c_float, c_int, c_int32, c_int64, c_uint64,
                    c_void_p)

import torch

_PKG_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# RSWA_LIBRARY lets a deployment point at a library built elsewhere.
LIB_PATH = os.environ.get("RSWA_LIBRARY") or os.path.join(_PKG_ROOT, "lib", "librswa.so")

RSWA_BF16, RSWA_F16, RSWA_F32, RSWA_F64 = 0, 1, 2, 3
_DTYPES = {
    torch.bfloat16: RSWA_BF16,
    torch.float16: RSWA_F16,
    torch.float32: RSWA_F32,
    torch.float64: RSWA_F64,
}

_I64x3 = c_int64 * 3
_I64x4 = c_int64 * 4


class AttnParams(Structure):
    """Mirror of ``rswa_attn_params`` (include/rswa.h); field order is the ABI."""

    _fields_ = [
        ("dtype", c_int32),
        ("head_dim", c_int32),
        ("batch", c_int32),
        ("heads_q", c_int32),
        ("heads_kv", c_int32),
        ("seqlen_q", c_int32),
        ("seqlen_k", c_int32),
        ("total_q", c_int64),
        ("total_k", c_int64),
        ("cu_seqlens_q", c_void_p),
        ("cu_seqlens_k", c_void_p),
        ("softmax_scale", c_float),
        ("window_left", c_int32),
        ("window_right", c_int32),
        ("causal", c_int32),
        ("num_sink", c_int32),
        ("shift_explicit", c_int32),
        ("shift", c_int32),
        ("q", c_void_p),
        ("k", c_void_p),
        ("v", c_void_p),
        ("q_stride", _I64x3),
        ("k_stride", _I64x3),
        ("v_stride", _I64x3),
        ("out", c_void_p),
        ("out_stride", _I64x3),
        ("lse", c_void_p),
        ("lse_stride", _I64x3),
        ("dout", c_void_p),
        ("dout_stride", _I64x3),
        ("dq", c_void_p),
        ("dk", c_void_p),
        ("dv", c_void_p),
        ("dq_stride", _I64x3),
        ("dk_stride", _I64x3),
        ("dv_stride", _I64x3),
        ("workspace", c_void_p),
        ("workspace_bytes", c_uint64),
        ("dq_accumulate", c_int32),
        ("addressing", c_int32),
        ("out_accumulate", c_int32),
        ("seg_rows", c_int32),
        ("k2", c_void_p),
        ("v2", c_void_p),
        ("dk2", c_void_p),
        ("dv2", c_void_p),
        ("ds_handoff", c_int32),
        ("wide", c_int32),
        ("dkv_accumulate", c_int32),
    ]

WIDE_OUT, WIDE_DQ, WIDE_DKV = 1, 2, 4


class RswaError(RuntimeError):
    pass


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with "
            f"`python {os.path.join(_PKG_ROOT, 'build.py')}` (needs hipcc; no GPU required). "
            "ring_swa has no non-HIP fallback."
        )
    _lib = load(LIB_PATH)
    return _lib


def load(path: str) -> ctypes.CDLL:
    """Open a build of the library and declare its entry points."""
    L = ctypes.CDLL(path)
    L.rswa_last_error.restype = c_char_p
    L.rswa_last_error.argtypes = []
    L.rswa_version.restype = c_int
    L.rswa_sizeof_attn_params.restype = c_uint64
    L.rswa_merge_attn_out.restype = c_int
    L.rswa_merge_attn_out.argtypes = [
        c_void_p, c_int, POINTER(c_int64),
        c_void_p, c_int, POINTER(c_int64),
        c_void_p, c_int, POINTER(c_int64),
        c_void_p, c_int, POINTER(c_int64),
        c_int64, c_int64, c_int64, c_int64, c_void_p,
    ]
    L.rswa_stream_copy.restype = c_int
    L.rswa_stream_copy.argtypes = [c_void_p, c_void_p, c_uint64, c_void_p]
    for name in ("rswa_attn_fwd", "rswa_attn_bwd", "rswa_attn_bwd_static"):
        fn = getattr(L, name)
        fn.restype = c_int
        fn.argtypes = [POINTER(AttnParams), c_void_p]
    L.rswa_attn_bwd_static_init.restype = c_int
    L.rswa_attn_bwd_static_init.argtypes = []
    L.rswa_attn_bwd_phases.restype = c_int
    L.rswa_attn_bwd_phases.argtypes = [POINTER(AttnParams), c_void_p, c_int]
    L.rswa_attn_bwd_workspace_bytes.restype = c_uint64
    L.rswa_attn_bwd_workspace_bytes.argtypes = [POINTER(AttnParams)]
    L.rswa_attn_bwd_handoff_active.restype = c_int
    L.rswa_attn_bwd_handoff_active.argtypes = [POINTER(AttnParams)]
    if L.rswa_sizeof_attn_params() != ctypes.sizeof(AttnParams):
        raise ImportError(
            "rswa_attn_params layout mismatch between librswa.so "
            f"({L.rswa_sizeof_attn_params()} bytes) and the Python binding "
            f"({ctypes.sizeof(AttnParams)} bytes): rebuild the library"
        )
    return L


def check(status: int) -> None:
    if status != 0:
        msg = lib().rswa_last_error().decode("utf-8", "replace")
        if status == -1:
            raise ValueError(msg)
        if status == -2:
            raise NotImplementedError(msg)
        raise RswaError(f"rswa status {status}: {msg}")


def dtype_code(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise NotImplementedError(f"unsupported dtype {t.dtype}") from None


def stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def require_device(*tensors: torch.Tensor) -> torch.device:
    dev = tensors[0].device
    if dev.type != "cuda":
        raise RuntimeError(
            "ring_swa kernels run on a ROCm GPU only (got a tensor on "
            f"'{dev}'); there is no CPU path"
        )
    for t in tensors:
        if t.device != dev:
            raise RuntimeError("all tensors must live on the same device")
    return dev


def i64x3(vals) -> _I64x3:
    return _I64x3(*[int(v) for v in vals])


def i64x4(vals) -> _I64x4:
    return _I64x4(*[int(v) for v in vals])
