"""GPU parity of the HIP backward attention kernels (through the C ABI) against
the CPU oracle.  Tolerance stated for this path: dQ, dK, dV within 5e-2 in
relative norm ||x - ref|| / ||ref||; the tests hold the kernels to 1e-2 plus an
elementwise bound (tests/gradcheck_util.py)."""
import itertools

import pytest
import torch

from oracle import attention_oracle as O

pytestmark = pytest.mark.gpu

from gradcheck_util import GRAD_TOL, relnorm as _relnorm  # noqa: E402


def _rand(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g).to(dtype)


def _run_dense(q, k, v, do, scale, window, causal, ns):
    """fwd + bwd on the GPU kernels, dq/dk/dv into fresh buffers."""
    from ring_swa.ops import wrapped_flash_attn_bwd, wrapped_flash_attn_fwd

    dq_, dk_, dv_, ddo = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    out, lse = wrapped_flash_attn_fwd(dq_, dk_, dv_, scale, window, causal, num_sink=ns)
    gq = torch.full_like(dq_, float("nan"))
    gk = torch.full_like(dk_, float("nan"))
    gv = torch.full_like(dv_, float("nan"))
    wrapped_flash_attn_bwd(dq_, dk_, dv_, out, lse, ddo, gq, gk, gv, scale, window, causal,
                           num_sink=ns)
    torch.cuda.synchronize()
    return out, lse, gq, gk, gv


DENSE_CASES = [
    # (B, Sq, Sk, Hq, Hkv, D, window, causal, n_sink)
    (1, 100, 100, 8, 2, 64, (50, 50), False, 0),     # test/test_local_swa.py:98-141
    (1, 1024, 1024, 8, 2, 64, (128, 0), True, 1),    # test/test_local_slm.py:76-119
    (2, 300, 300, 4, 4, 128, (37, 0), True, 0),
    (1, 257, 257, 4, 1, 128, (-1, -1), False, 0),
    (1, 130, 130, 2, 2, 128, (0, 0), True, 0),
    (1, 200, 333, 4, 2, 128, (40, 0), True, 0),
    (1, 333, 200, 4, 2, 128, (40, 0), True, 0),      # leading rows see nothing
    (1, 96, 160, 2, 1, 128, (0, 4096), False, 0),
    (1, 160, 160, 2, 1, 128, (70, 160), False, 0),
    (1, 190, 64, 2, 1, 128, (10, 4096), False, 0),
    (2, 700, 700, 4, 2, 128, (100, 0), True, 4),
    (1, 513, 513, 2, 2, 128, (1000, 0), True, 2),
    (1, 2048, 2048, 4, 2, 128, (500, 0), True, 0),
    (1, 1, 1, 1, 1, 128, (5, 0), True, 0),
    # sink keys under a bounded window: their dK / dV rows come from the sink kernel, in
    # passes of four keys -- one pass partly filled, several passes, sinks across two key tiles,
    # more sinks than keys, queries aligned to the end of a longer key range, two-sided window
    (1, 900, 900, 4, 2, 128, (64, 0), True, 3),
    (1, 1200, 1200, 6, 2, 64, (100, 0), True, 9),
    (2, 1500, 1500, 2, 1, 128, (32, 0), True, 70),
    (1, 1100, 1100, 4, 4, 64, (16, 0), True, 300),
    (1, 40, 40, 2, 1, 128, (3, 0), True, 64),
    (1, 300, 800, 4, 2, 128, (50, 0), True, 5),
    (1, 600, 600, 2, 2, 64, (30, 20), False, 6),
]


@pytest.mark.parametrize("case", DENSE_CASES, ids=lambda c: "x".join(str(x) for x in c))
def test_bwd_dense_matches_oracle(case):
    b, sq, sk, hq, hk, d, window, causal, ns = case
    q = _rand((b, sq, hq, d), torch.bfloat16, 1)
    k = _rand((b, sk, hk, d), torch.bfloat16, 2)
    v = _rand((b, sk, hk, d), torch.bfloat16, 3)
    do = _rand((b, sq, hq, d), torch.bfloat16, 4)
    scale = d ** -0.5
    _, _, rq, rk, rv = O.attention_fwd_bwd(
        lambda q, k, v: O.window_attention(q, k, v, scale, window, causal, ns), q, k, v, do
    )
    out, lse, gq, gk, gv = _run_dense(q, k, v, do, scale, window, causal, ns)
    errs = [_relnorm(g, r) for g, r in ((gq, rq), (gk, rk), (gv, rv))]
    assert max(errs) <= GRAD_TOL, f"rel-norm errors dq/dk/dv = {errs}"


def test_bwd_with_ones_upstream_like_the_reference_test():
    """dO = ones, GQA 4:1, two-sided window — the check of test/test_local_swa.py:129-141."""
    q = _rand((1, 100, 8, 64), torch.bfloat16, 42)
    k = _rand((1, 100, 2, 64), torch.bfloat16, 43)
    v = _rand((1, 100, 2, 64), torch.bfloat16, 44)
    do = torch.ones(1, 100, 8, 64, dtype=torch.bfloat16)
    _, _, rq, rk, rv = O.attention_fwd_bwd(
        lambda q, k, v: O.window_attention(q, k, v, None, (50, 50), False), q, k, v, do
    )
    _, _, gq, gk, gv = _run_dense(q, k, v, do, 64 ** -0.5, (50, 50), False, 0)
    for g, r in ((gq, rq), (gk, rk), (gv, rv)):
        # the reference asserts atol = rtol = 1e-2 on bf16 gradients
        bad = (g.float().cpu() - r).abs() > 1e-2 + 1e-2 * r.abs()
        assert bad.float().mean().item() < 1e-2, "too many elements outside atol=rtol=1e-2"
        assert _relnorm(g, r) <= GRAD_TOL


def test_bwd_uses_the_callers_merged_statistics():
    """Keys split in two blocks, each backward fed the FINAL (o, lse): the sum equals
    the gradient of attention over all keys (ring_swa/sliding_window/nonvarlen.py:242-253)."""
    from ring_swa.ops import merge_attn_out, wrapped_flash_attn_bwd, wrapped_flash_attn_fwd

    b, s, hq, hk, d, w = 1, 384, 4, 2, 128, 200
    q = _rand((b, s, hq, d), torch.bfloat16, 1)
    k = _rand((b, 2 * s, hk, d), torch.bfloat16, 2)
    v = _rand((b, 2 * s, hk, d), torch.bfloat16, 3)
    do = _rand((b, s, hq, d), torch.bfloat16, 4)
    # queries are the last s positions of a 2s-long sequence, window w: keys split at s
    _, _, rq, rk, rv = O.attention_fwd_bwd(
        lambda q, k, v: O.window_attention(q, k, v, None, (w, 0), True), q, k, v, do
    )
    dq_, dk_, dv_, ddo = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    # block A: own chunk (causal band); block B: previous chunk, upper-right triangle
    oa, la = wrapped_flash_attn_fwd(dq_, dk_[:, s:], dv_[:, s:], None, (w, 0), True)
    ob, lb = wrapped_flash_attn_fwd(dq_[:, :w], dk_[:, s - w:s], dv_[:, s - w:s], None, (0, s), False)
    acc = oa.float()
    lacc = la.clone()
    merge_attn_out(acc[:, :w], lacc[:, :, :w], ob, lb)
    o_fin = acc.to(torch.bfloat16)
    gq = torch.zeros_like(dq_, dtype=torch.float32)
    gk = torch.zeros_like(dk_, dtype=torch.float32)
    gv = torch.zeros_like(dv_, dtype=torch.float32)
    tq, tk, tv = torch.empty_like(dq_), torch.empty_like(dk_[:, s:]), torch.empty_like(dv_[:, s:])
    wrapped_flash_attn_bwd(dq_, dk_[:, s:], dv_[:, s:], o_fin, lacc, ddo, tq, tk, tv, None, (w, 0), True)
    gq += tq
    gk[:, s:] += tk
    gv[:, s:] += tv
    tq2 = torch.empty_like(dq_[:, :w])
    tk2, tv2 = torch.empty_like(dk_[:, s - w:s]), torch.empty_like(dv_[:, s - w:s])
    wrapped_flash_attn_bwd(dq_[:, :w], dk_[:, s - w:s], dv_[:, s - w:s], o_fin[:, :w],
                           lacc[:, :, :w].contiguous(), ddo[:, :w], tq2, tk2, tv2, None, (0, s), False)
    gq[:, :w] += tq2
    gk[:, s - w:s] += tk2
    gv[:, s - w:s] += tv2
    torch.cuda.synchronize()
    errs = [_relnorm(g, r) for g, r in ((gq, rq), (gk, rk), (gv, rv))]
    assert max(errs) <= GRAD_TOL, f"rel-norm errors dq/dk/dv = {errs}"


def test_bwd_into_strided_views():
    """dq/dk/dv handed in as slices of larger buffers (ring_swa/streaming_llm/naive.py:53-66)."""
    from ring_swa.ops import wrapped_flash_attn_bwd, wrapped_flash_attn_fwd

    q = _rand((2, 201, 4, 128), torch.bfloat16, 1)
    k = _rand((2, 201, 2, 128), torch.bfloat16, 2)
    v = _rand((2, 201, 2, 128), torch.bfloat16, 3)
    do = _rand((2, 201, 4, 128), torch.bfloat16, 4)
    _, _, rq, rk, rv = O.attention_fwd_bwd(
        lambda q, k, v: O.window_attention(q, k, v, None, (20, 0), True),
        q[:, 1:], k[:, 1:], v[:, 1:], do[:, 1:],
    )
    dq_, dk_, dv_, ddo = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    o, lse = wrapped_flash_attn_fwd(dq_[:, 1:], dk_[:, 1:], dv_[:, 1:], None, (20, 0), True)
    gq, gk, gv = torch.zeros_like(dq_), torch.zeros_like(dk_), torch.zeros_like(dv_)
    wrapped_flash_attn_bwd(dq_[:, 1:], dk_[:, 1:], dv_[:, 1:], o, lse, ddo[:, 1:], gq[:, 1:],
                           gk[:, 1:], gv[:, 1:], None, (20, 0), True)
    torch.cuda.synchronize()
    assert torch.all(gq[:, 0] == 0) and torch.all(gk[:, 0] == 0) and torch.all(gv[:, 0] == 0)
    errs = [_relnorm(g[:, 1:], r) for g, r in ((gq, rq), (gk, rk), (gv, rv))]
    assert max(errs) <= GRAD_TOL, f"rel-norm errors dq/dk/dv = {errs}"


@pytest.mark.parametrize("lens,window,ns", [
    ([5, 130, 64, 1, 300], (50, 0), 0),
    ([257, 255], (-1, 0), 0),
    ([100, 400, 129], (64, 0), 4),
    ([3, 700, 1, 260, 2000], (40, 0), 7),
])
def test_bwd_varlen_matches_oracle(lens, window, ns):
    from ring_swa.ops import wrapped_flash_attn_bwd_varlen, wrapped_flash_attn_fwd_varlen

    cu = torch.tensor([0] + list(itertools.accumulate(lens)), dtype=torch.int32)
    t = int(cu[-1])
    q = _rand((t, 4, 128), torch.bfloat16, 1)
    k = _rand((t, 2, 128), torch.bfloat16, 2)
    v = _rand((t, 2, 128), torch.bfloat16, 3)
    do = _rand((t, 4, 128), torch.bfloat16, 4)
    _, _, rq, rk, rv = O.attention_fwd_bwd(
        lambda q, k, v: O.window_attention_varlen(q, k, v, cu, cu, None, window, True, ns),
        q, k, v, do,
    )
    dq_, dk_, dv_, ddo, dcu = q.cuda(), k.cuda(), v.cuda(), do.cuda(), cu.cuda()
    o, lse = wrapped_flash_attn_fwd_varlen(dq_, dk_, dv_, None, window, dcu, dcu, None, None, True,
                                           num_sink=ns)
    gq, gk, gv = torch.empty_like(dq_), torch.empty_like(dk_), torch.empty_like(dv_)
    wrapped_flash_attn_bwd_varlen(dq_, dk_, dv_, o, lse, ddo, gq, gk, gv, None, window, dcu, dcu,
                                  None, None, True, num_sink=ns)
    torch.cuda.synchronize()
    errs = [_relnorm(g, r) for g, r in ((gq, rq), (gk, rk), (gv, rv))]
    assert max(errs) <= GRAD_TOL, f"rel-norm errors dq/dk/dv = {errs}"


def test_bwd_varlen_one_key_per_sequence():
    """The per-sequence sink backward of ring_swa/streaming_llm/naive.py:181-206: every
    sequence attends one key of its own (cu_seqlens_k = arange)."""
    from ring_swa.ops import wrapped_flash_attn_bwd_varlen, wrapped_flash_attn_fwd_varlen

    lens_q = [70, 200, 3]
    cu_q = torch.tensor([0] + list(itertools.accumulate(lens_q)), dtype=torch.int32)
    cu_k = torch.arange(0, 4, dtype=torch.int32)
    t = int(cu_q[-1])
    q = _rand((t, 4, 128), torch.bfloat16, 1)
    k = _rand((3, 2, 128), torch.bfloat16, 2)
    v = _rand((3, 2, 128), torch.bfloat16, 3)
    do = _rand((t, 4, 128), torch.bfloat16, 4)
    _, _, rq, rk, rv = O.attention_fwd_bwd(
        lambda q, k, v: O.window_attention_varlen(q, k, v, cu_q, cu_k, None, (-1, -1), False),
        q, k, v, do,
    )
    dq_, dk_, dv_, ddo = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    o, lse = wrapped_flash_attn_fwd_varlen(dq_, dk_, dv_, None, (-1, -1), cu_q.cuda(), cu_k.cuda(),
                                           200, 1, False)
    gq, gk, gv = torch.empty_like(dq_), torch.empty_like(dk_), torch.empty_like(dv_)
    wrapped_flash_attn_bwd_varlen(dq_, dk_, dv_, o, lse, ddo, gq, gk, gv, None, (-1, -1),
                                  cu_q.cuda(), cu_k.cuda(), 200, 1, False)
    torch.cuda.synchronize()
    # softmax over a single key is constant: dq and dk vanish, dv is the column sum of dO
    assert gq.abs().max().item() <= 1e-2 and gk.abs().max().item() <= 1e-2
    assert _relnorm(gv, rv) <= GRAD_TOL


def test_bwd_fp16():
    q = _rand((1, 150, 4, 128), torch.float16, 1)
    k = _rand((1, 150, 2, 128), torch.float16, 2)
    v = _rand((1, 150, 2, 128), torch.float16, 3)
    do = _rand((1, 150, 4, 128), torch.float16, 4)
    _, _, rq, rk, rv = O.attention_fwd_bwd(
        lambda q, k, v: O.window_attention(q, k, v, 0.2, (33, 0), True), q, k, v, do
    )
    _, _, gq, gk, gv = _run_dense(q, k, v, do, 0.2, (33, 0), True, 0)
    errs = [_relnorm(g, r) for g, r in ((gq, rq), (gk, rk), (gv, rv))]
    assert max(errs) <= GRAD_TOL, f"rel-norm errors dq/dk/dv = {errs}"


@pytest.mark.parametrize("hq,hk,s", [(4, 2, 300), (3, 3, 257)])
def test_bwd_dq_accumulate_is_one_fp32_add_of_the_two_16bit_values(hq, hk, s):
    """dq_accumulate: dq <- round(float(dq) + float(round(dQ))), bit for bit; dk / dv as
    without it.  Also with the phases of one backward spread over two calls, as the
    two-block ring step uses them."""
    from ring_swa.ops import attn_bwd, attn_fwd
    from ring_swa.ops.band_attn import bwd_workspace_bytes

    g = torch.Generator().manual_seed(7)
    q, do = (torch.randn(2, s, hq, 128, generator=g).bfloat16().cuda() for _ in range(2))
    k, v = (torch.randn(2, s, hk, 128, generator=g).bfloat16().cuda() for _ in range(2))
    base = torch.randn(2, s, hq, 128, generator=g).bfloat16().cuda()
    out, lse = attn_fwd(q, k, v, None, (100, 0), True)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    attn_bwd(q, k, v, out, lse, do, dq, dk, dv, None, (100, 0), True)
    acc, dk2, dv2 = base.clone(), torch.empty_like(k), torch.empty_like(v)
    ws = torch.empty(bwd_workspace_bytes(q, k), dtype=torch.uint8, device="cuda")
    attn_bwd(q, k, v, out, lse, do, acc, dk2, dv2, None, (100, 0), True, workspace=ws, phases=3)
    assert torch.equal(acc, base)  # the dQ kernel has not run yet
    attn_bwd(q, k, v, out, lse, do, acc, dk2, dv2, None, (100, 0), True, workspace=ws, phases=4,
             dq_accumulate=True)
    torch.cuda.synchronize()
    assert torch.equal(acc, (base.float() + dq.float()).bfloat16())
    assert torch.equal(dk2, dk) and torch.equal(dv2, dv)


@pytest.mark.parametrize("sq,sk,hq,hk,d,window", [
    (300, 1000, 4, 4, 64, (-1, -1)),   # 2*300*4 statistics: 32 elements short of 256 bytes
    (301, 301, 3, 1, 128, (50, 0)),
    (77, 500, 5, 5, 128, (20, 0)),
])
def test_bwd_does_not_depend_on_what_the_workspace_held(sq, sk, hq, hk, d, window):
    """The statistics arrays in the workspace are padded to 256 bytes and the tile kernels read
    a tile of rows past a sequence's last one: whatever the caller's workspace held before (NaN
    here, +inf, zeros) the results are the same bits."""
    from ring_swa.ops import attn_bwd, attn_fwd
    from ring_swa.ops.band_attn import bwd_workspace_bytes

    g = torch.Generator().manual_seed(11)
    q, do = (torch.randn(2, sq, hq, d, generator=g).bfloat16().cuda() for _ in range(2))
    k, v = (torch.randn(2, sk, hk, d, generator=g).bfloat16().cuda() for _ in range(2))
    out, lse = attn_fwd(q, k, v, None, window, True)
    results = []
    for fill in (float("nan"), float("inf"), 0.0):
        ws = torch.full((bwd_workspace_bytes(q, k) // 4,), fill, device="cuda").view(torch.uint8)
        dq, dk, dv = (torch.full_like(t, float("nan")) for t in (q, k, v))
        attn_bwd(q, k, v, out, lse, do, dq, dk, dv, None, window, True, workspace=ws)
        results.append((dq, dk, dv))
    for dq, dk, dv in results:
        for name, x, y in zip(("dq", "dk", "dv"), (dq, dk, dv), results[-1]):
            assert torch.isfinite(x.float()).all(), name
            assert torch.equal(x, y), name


def test_bwd_empty_queries_write_only_the_outputs_of_the_requested_phases():
    """No query rows: dK = dV = 0 and dQ is empty, but a call restricted to the dQ phase
    must leave dK / dV (another call's results) alone."""
    from ring_swa.ops import attn_bwd

    q = torch.empty(1, 0, 4, 128, dtype=torch.bfloat16, device="cuda")
    k = _rand((1, 96, 2, 128), torch.bfloat16, 2).cuda()
    v = _rand((1, 96, 2, 128), torch.bfloat16, 3).cuda()
    o, do, dq = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
    lse = torch.empty(1, 4, 0, dtype=torch.float32, device="cuda")
    dk, dv = torch.full_like(k, 7.0), torch.full_like(v, 7.0)
    attn_bwd(q, k, v, o, lse, do, dq, dk, dv, None, (16, 0), True, phases=1 | 4)
    assert bool((dk == 7).all()) and bool((dv == 7).all())
    attn_bwd(q, k, v, o, lse, do, dq, dk, dv, None, (16, 0), True)
    assert bool((dk == 0).all()) and bool((dv == 0).all())


def test_bwd_packed_with_trailing_pad_rows_full_of_nan():
    """A pack shorter than its buffers (total rows > cu_seqlens[-1]): the rows behind the last
    sequence belong to nobody and hold NaN in q, k, v, out and dout.  Nothing of that may
    reach the gradients of the real rows: the last query tile of a sequence reads the
    statistics of the rows that follow it, and 0 * NaN would be NaN."""
    from ring_swa.ops import attn_bwd, attn_fwd

    hq, hk, d, w = 4, 2, 128, 40
    cu = [0, 70, 199, 200, 333]
    total, pad = cu[-1], 60
    q = _rand((total, hq, d), torch.bfloat16, 1)
    k = _rand((total, hk, d), torch.bfloat16, 2)
    v = _rand((total, hk, d), torch.bfloat16, 3)
    do = _rand((total, hq, d), torch.bfloat16, 4)
    _, _, rq, rk, rv = O.attention_fwd_bwd(
        lambda q, k, v: O.window_attention_varlen(q, k, v, cu, cu, None, (w, 0), True), q, k, v, do)

    def padded(t):
        buf = torch.full((total + pad, *t.shape[1:]), float("nan"), dtype=t.dtype, device="cuda")
        buf[:total] = t.cuda()
        return buf

    qp, kp, vp, dop = padded(q), padded(k), padded(v), padded(do)
    cud = torch.tensor(cu, dtype=torch.int32, device="cuda")
    out, lse = attn_fwd(qp, kp, vp, None, (w, 0), True, cud, cud)
    out[total:] = float("nan")
    lse[:, total:] = float("nan")
    gq, gk, gv = (torch.full_like(t, 5.0) for t in (qp, kp, vp))
    attn_bwd(qp, kp, vp, out, lse, dop, gq, gk, gv, None, (w, 0), True, cud, cud)
    torch.cuda.synchronize()
    errs = [_relnorm(g[:total], r) for g, r in ((gq, rq), (gk, rk), (gv, rv))]
    assert max(errs) <= GRAD_TOL, f"rel-norm errors dq/dk/dv = {errs}"


def test_bwd_accepts_plus_inf_lse_for_empty_rows():
    """flash-attn marks rows without any visible key with lse = +inf, this library with -inf
    (the merge identity).  A caller that hands in +inf gets the same gradients: P is zero for
    such rows either way."""
    from ring_swa.ops import attn_bwd, attn_fwd

    # 333 queries against 200 keys, bottom-right aligned: the first 133 rows see nothing
    q = _rand((1, 333, 4, 128), torch.bfloat16, 1).cuda()
    k = _rand((1, 200, 2, 128), torch.bfloat16, 2).cuda()
    v = _rand((1, 200, 2, 128), torch.bfloat16, 3).cuda()
    do = _rand((1, 333, 4, 128), torch.bfloat16, 4).cuda()
    out, lse = attn_fwd(q, k, v, None, (40, 0), True)
    assert torch.isinf(lse[:, :, :133]).all() and (lse[:, :, :133] < 0).all()
    assert (out[:, :133] == 0).all()
    a = [torch.empty_like(t) for t in (q, k, v)]
    b = [torch.empty_like(t) for t in (q, k, v)]
    attn_bwd(q, k, v, out, lse, do, *a, None, (40, 0), True)
    lse_pos = torch.where(torch.isinf(lse), torch.full_like(lse, float("inf")), lse)
    attn_bwd(q, k, v, out, lse_pos, do, *b, None, (40, 0), True)
    torch.cuda.synchronize()
    for x, y in zip(a, b):
        assert torch.isfinite(x.float()).all()
        assert torch.equal(x, y)
