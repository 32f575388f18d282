"""CPU-side checks of the C-ABI boundary: the library loads, exports every
symbol the header declares, the Python struct mirrors the C struct, and
argument validation fails cleanly without touching a GPU."""
import ctypes
import importlib.util
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "ring-sliding-window-attention_amd")
HEADER = os.path.join(ROOT, "include", "rswa.h")


def _ensure_built():
    lib = os.path.join(PKG, "lib", "librswa.so")
    if not os.path.exists(lib):
        spec = importlib.util.spec_from_file_location("rswa_build", os.path.join(PKG, "build.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        mod.build()
    return lib


def _declared_symbols():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(rswa_[a-z_0-9]+)\s*\(", src)))


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_ensure_built())
    names = _declared_symbols()
    assert {"rswa_merge_attn_out", "rswa_attn_fwd", "rswa_attn_bwd", "rswa_last_error",
            "rswa_attn_bwd_workspace_bytes"} <= set(names)
    for n in names:
        assert hasattr(lib, n), f"librswa.so does not export {n}"


def test_python_struct_matches_c_struct():
    _ensure_built()
    from ring_swa import _lib

    L = _lib.lib()
    assert L.rswa_sizeof_attn_params() == ctypes.sizeof(_lib.AttnParams)
    assert L.rswa_version() == 3


def test_header_cites_reference_interfaces():
    src = open(HEADER).read()
    for cite in ("ring_swa/ops/merge.py:150", "ring_swa/ops/wrap_flash.py:168",
                 "ring_swa/ops/wrap_flash.py:276"):
        assert cite in src


def test_merge_argument_validation_needs_no_gpu():
    _ensure_built()
    from ring_swa import _lib

    L = _lib.lib()
    st4 = _lib.i64x4((8 * 4 * 128, 4 * 128, 128, 1))
    st3 = _lib.i64x3((4 * 8, 8, 1))
    # head_dim not a multiple of 8 -> unsupported, reported through rswa_last_error
    rc = L.rswa_merge_attn_out(16, 2, st4, 16, 2, st3, 16, 0, st4, 16, 2, st3, 1, 8, 4, 100, None)
    assert rc == -2 and b"head_dim" in L.rswa_last_error()
    # null tensor -> invalid
    rc = L.rswa_merge_attn_out(None, 2, st4, 16, 2, st3, 16, 0, st4, 16, 2, st3, 1, 8, 4, 128, None)
    assert rc == -1
    # empty problem is a no-op
    rc = L.rswa_merge_attn_out(None, 2, st4, None, 2, st3, None, 0, st4, None, 2, st3, 0, 8, 4, 128,
                               None)
    assert rc == 0


def test_ops_refuse_cpu_tensors():
    _ensure_built()
    from ring_swa.ops import merge_attn_out

    o = torch.zeros(1, 8, 2, 128)
    l = torch.zeros(1, 2, 8)
    with pytest.raises(RuntimeError, match="no CPU path"):
        merge_attn_out(o, l, o.clone(), l.clone())


def test_static_backward_refuses_oversize_without_a_gpu():
    _ensure_built()
    from ring_swa import _lib

    L = _lib.lib()
    p = _lib.AttnParams()
    p.dtype, p.head_dim, p.batch, p.heads_q, p.heads_kv = 0, 128, 1, 32, 8
    p.seqlen_q, p.seqlen_k = 131073, 8  # one row more than the built-in buffer serves
    p.softmax_scale = 1.0
    assert L.rswa_attn_bwd_workspace_bytes(p) > (32 << 20)
    rc = L.rswa_attn_bwd_static(p, None)
    assert rc == -2 and b"built-in" in L.rswa_last_error()
    assert L.rswa_attn_bwd_static(None, None) == -1


def _fake_params(tokens, heads_q=32, heads_kv=8, d=128):
    """Dense one-batch problem on placeholder addresses: enough for the argument checks,
    which run before anything touches a device."""
    from ring_swa import _lib

    p = _lib.AttnParams()
    p.dtype, p.head_dim, p.batch, p.heads_q, p.heads_kv = 0, d, 1, heads_q, heads_kv
    p.seqlen_q = p.seqlen_k = tokens
    p.softmax_scale = d ** -0.5
    p.window_left, p.window_right, p.causal = 1024, 0, 1
    for name in ("q", "k", "v", "out", "lse", "dout", "dq", "dk", "dv", "workspace"):
        setattr(p, name, 4096)
    rq, rk = (heads_q * d, d), (heads_kv * d, d)
    for name, (row, head) in (("q", rq), ("k", rk), ("v", rk), ("out", rq), ("dout", rq),
                              ("dq", rq), ("dk", rk), ("dv", rk)):
        setattr(p, name + "_stride", _lib.i64x3((tokens * row, row, head)))
    p.lse_stride = _lib.i64x3((heads_q * tokens, tokens, 1))
    return p


def test_what_stays_refused_beyond_2_gib_says_why():
    """A sequence may span any number of bytes; what the 32-bit tile offsets still cannot
    serve is refused with a message that names the limit."""
    _ensure_built()
    from ring_swa import _lib

    L = _lib.lib()
    # rows 4 MiB apart: one 256-row tile would span 2 GiB
    p = _fake_params(1024)
    p.k_stride = _lib.i64x3((0, 1 << 22, 128))
    assert L.rswa_attn_fwd(p, None) == -2
    assert b"row stride" in L.rswa_last_error()
    p = _fake_params(1024)
    p.dout_stride = _lib.i64x3((0, 1 << 22, 128))
    p.workspace_bytes = L.rswa_attn_bwd_workspace_bytes(p)
    assert L.rswa_attn_bwd(p, None) == -2
    assert b"row stride of dout" in L.rswa_last_error()
    # 2^24 + ... rows x 32 heads: each statistics array of the backward would reach 2 GiB
    p = _fake_params(1 << 24)
    p.workspace_bytes = L.rswa_attn_bwd_workspace_bytes(p)
    assert L.rswa_attn_bwd(p, None) == -2
    assert b"statistics array" in L.rswa_last_error()
    # a little below that limit passes the size checks: the workspace is next
    p = _fake_params((1 << 24) - 1024)
    p.workspace_bytes = 0
    assert L.rswa_attn_bwd(p, None) == -1
    assert b"workspace" in L.rswa_last_error()


def test_mask_arithmetic_limits_are_refused_or_mapped():
    """The kernels compute masks in 32 bits: an explicit shift of 2^28 or more and sequences
    that long are refused with a message; a window that reaches that far is the unbounded one
    (the argument checks run before anything touches a device)."""
    _ensure_built()
    from ring_swa import _lib

    L = _lib.lib()
    p = _fake_params(1024)
    p.shift_explicit, p.shift = 1, 1 << 28
    assert L.rswa_attn_fwd(p, None) == -2
    assert b"shift" in L.rswa_last_error()
    p.shift = -(1 << 28)
    assert L.rswa_attn_fwd(p, None) == -2
    p = _fake_params(1 << 28, heads_q=1, heads_kv=1)
    assert L.rswa_attn_fwd(p, None) == -2
    assert b"2^28" in L.rswa_last_error()
    # a window of 2^30 keys is accepted (it is the unbounded window): the backward's checks go
    # on to the workspace
    p = _fake_params(1024)
    p.window_left = 1 << 30
    p.workspace_bytes = 0
    assert L.rswa_attn_bwd(p, None) == -1
    assert b"workspace" in L.rswa_last_error()


def test_two_key_ranges_are_checked_before_any_launch():
    """seg_rows splits the key rows over (k, v) and (k2, v2): dense problems without sink keys,
    a boundary that is a positive multiple of 256 below seqlen_k, and the second range's
    tensors present (dk2 / dv2 too for the backward)."""
    _ensure_built()
    from ring_swa import _lib

    L = _lib.lib()

    def params(seg=512, **kw):
        p = _fake_params(1024)
        p.seg_rows = seg
        p.k2 = p.v2 = p.dk2 = p.dv2 = 8192
        for key, val in kw.items():
            setattr(p, key, val)
        return p

    for bad in (100, -256, 1024, 1280):
        assert L.rswa_attn_fwd(params(bad), None) == -2, bad
        assert b"seg_rows" in L.rswa_last_error()
    assert L.rswa_attn_fwd(params(num_sink=2), None) == -2
    assert b"sink" in L.rswa_last_error()
    assert L.rswa_attn_fwd(params(k2=0), None) == -1
    assert b"k2" in L.rswa_last_error()
    assert L.rswa_attn_fwd(params(v2=8), None) == -2       # not 16-byte aligned
    p = params(dk2=0)
    p.workspace_bytes = 1 << 30
    assert L.rswa_attn_bwd(p, None) == -1
    assert b"dk2" in L.rswa_last_error()
    # a well-formed pair of ranges passes these checks: the backward goes on to the workspace
    p = params()
    p.workspace_bytes = 0
    assert L.rswa_attn_bwd(p, None) == -1
    assert b"workspace" in L.rswa_last_error()
