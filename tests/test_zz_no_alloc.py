"""The allocation-free backward entry point (``rswa_attn_bwd_static``, statistics in the
library's own device buffer) gives what ``rswa_attn_bwd`` gives with a caller workspace: dQ
bit for bit, dK / dV to the last place (see ``_same``).  Two calls in a row, the second on a smaller input, so
that stale statistics of the first call would show; then a size beyond the buffer is refused.
Collected last on purpose (file name): a failure here must not hide the other tests."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _case(seed, b, s, hq, hk, d, window, packed_cu=None):
    g = torch.Generator().manual_seed(seed)
    if packed_cu is None:
        shape_q, shape_k = (b, s, hq, d), (b, s, hk, d)
    else:
        shape_q, shape_k = (s, hq, d), (s, hk, d)
    q, do = (torch.randn(*shape_q, generator=g).bfloat16().cuda() for _ in range(2))
    k, v = (torch.randn(*shape_k, generator=g).bfloat16().cuda() for _ in range(2))
    return q, k, v, do


def _both(q, k, v, do, window, cu=None, ns=0):
    from ring_swa.ops import attn_bwd, attn_fwd
    from ring_swa.ops.band_attn import bwd_static_init

    out, lse = attn_fwd(q, k, v, None, window, True, cu, cu, num_sink=ns)
    bwd_static_init()  # (the one-time address look-up may load the device image: not counted)
    grads = []
    for static in (False, True):
        dq, dk, dv = (torch.full_like(t, float("nan")) for t in (q, k, v))
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        free_before = torch.cuda.mem_get_info()[0]  # the device's own count: sees any hipMalloc
        attn_bwd(q, k, v, out, lse, do, dq, dk, dv, None, window, True, cu, cu, num_sink=ns,
                 static_workspace=static)
        torch.cuda.synchronize()
        if static:
            assert torch.cuda.memory_allocated() == before, "the static entry point allocated"
            assert torch.cuda.mem_get_info()[0] == free_before, (
                "device memory was allocated under the static entry point")
        grads.append((dq, dk, dv))
    return grads


def _same(with_workspace, static):
    """dQ bit for bit.  dK / dV: with a caller workspace the dK/dV kernel may deal the q heads of
    a GQA group to several blocks and add their fp32 partial sums at the end; on the built-in
    buffer it never does, so the fp32 sums are associated differently and the 16-bit results
    may differ in the last place of single entries (floating point: the path's tolerance is a
    relative norm of 5e-2; asserted here: one 16-bit unit in the last place)."""
    assert torch.equal(with_workspace[0], static[0])
    for x, y in zip(with_workspace[1:], static[1:]):
        assert not torch.isnan(y.float()).any()
        x, y = x.float(), y.float()
        # one unit in the last place of the entry, plus the fp32 reassociation error of sums
        # whose terms are as large as the tensor's largest entry (entries that nearly cancel)
        ulp = torch.maximum(x.abs(), y.abs()) * 2.0 ** -7 + 4e-6 * x.abs().max()
        assert ((x - y).abs() <= ulp).all()
        assert (x != y).float().mean().item() < 0.05


def test_static_backward_equals_workspace_backward_twice_in_a_row():
    # first call: 2 x 1536 rows x 8 heads; second, smaller: packed 700 rows x 4 heads
    q, k, v, do = _case(0, 2, 1536, 8, 2, 128, (200, 0))
    (a, b) = _both(q, k, v, do, (200, 0))
    _same(a, b)
    cu = torch.tensor([0, 130, 131, 500, 700], dtype=torch.int32, device="cuda")
    q, k, v, do = _case(1, 1, 700, 4, 4, 64, (64, 0), packed_cu=cu)
    (a, b) = _both(q, k, v, do, (64, 0), cu)
    _same(a, b)


def test_static_backward_with_sink_keys_under_a_bounded_window():
    """Then the sink kernel's arrival counters and fp32 sums live in the built-in buffer too
    (dense, then packed and smaller): the counters must come back to zero between the calls."""
    q, k, v, do = _case(2, 2, 1100, 8, 2, 128, (100, 0))
    k[:, :3] *= 4
    _same(*_both(q, k, v, do, (100, 0), ns=3))
    cu = torch.tensor([0, 300, 301, 900], dtype=torch.int32, device="cuda")
    q, k, v, do = _case(3, 1, 900, 4, 2, 64, (40, 0), packed_cu=cu)
    _same(*_both(q, k, v, do, (40, 0), cu, ns=5))
    _same(*_both(q, k, v, do, (40, 0), cu, ns=5))


def test_static_backward_replays_from_a_graph():
    """For callers under HIP graph capture: warm up (address look-up) outside the capture, capture
    one static backward, replay it with eager work in between, same bits as the eager call."""
    from ring_swa.ops import attn_bwd, attn_fwd
    from ring_swa.ops.band_attn import bwd_static_init

    q, k, v, do = _case(4, 1, 768, 8, 2, 128, (200, 0))
    out, lse = attn_fwd(q, k, v, None, (200, 0), True)
    dq, dk, dv = (torch.empty_like(t) for t in (q, k, v))
    run = lambda: attn_bwd(q, k, v, out, lse, do, dq, dk, dv, None, (200, 0), True,  # noqa: E731
                           static_workspace=True)
    bwd_static_init()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run()
    for trial in range(3):
        g = torch.Generator().manual_seed(20 + trial)
        do.copy_(torch.randn(do.shape, generator=g).bfloat16())
        for t in (dq, dk, dv):
            t.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in (dq, dk, dv)]
        run()  # eager work between the replays
        torch.cuda.synchronize()
        for a, b in zip(got, (dq, dk, dv)):
            assert torch.equal(a, b), f"replay {trial} differs from the eager call"


def test_static_backward_refuses_sizes_beyond_its_buffer():
    from ring_swa import _lib
    from ring_swa.ops import band_attn

    # 4 194 304 + 32 (row, head) pairs: one head row more than the buffer holds
    rows, heads = 131073, 32
    q = torch.empty(1, 8, heads, 128, dtype=torch.bfloat16, device="cuda")
    p = band_attn._params(q, q, q, 1.0, (8, 0), True, None, None, 0)
    p.seqlen_q = rows
    p.seqlen_k = 8
    for name in ("out", "lse", "dout", "dq", "dk", "dv"):
        setattr(p, name, q.data_ptr())
    st = _lib.i64x3((rows * heads * 128, heads * 128, 128))
    for name in ("out_stride", "dout_stride", "dq_stride", "dk_stride", "dv_stride"):
        setattr(p, name, st)
    p.lse_stride = _lib.i64x3((heads * rows, rows, 1))
    rc = _lib.lib().rswa_attn_bwd_static(p, None)
    assert rc == -2
    assert b"built-in" in _lib.lib().rswa_last_error()
