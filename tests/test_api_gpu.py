"""GPU parity of the public entry points (autograd included) against the CPU
oracle, plus the reference's own distributed invariant run on one GPU: the
concatenation of every virtual rank's share equals the single-call result
(test/test_ring_swa_nonvarlen.py:137-167, 218-229)."""
import itertools

import pytest
import torch

from oracle import attention_oracle as O

pytestmark = pytest.mark.gpu

from gradcheck_util import GRAD_TOL, relnorm as _relnorm  # noqa: E402

OUT_TOL = 2e-2


def _rand(shape, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g).to(dtype)


def _gpu_fwd_bwd(fn, q, k, v, do):
    q, k, v = (t.cuda().requires_grad_() for t in (q, k, v))
    out = fn(q, k, v)
    out.backward(do.cuda())
    torch.cuda.synchronize()
    return out.detach(), q.grad, k.grad, v.grad


def _compare(gpu, ref):
    out, dq, dk, dv = gpu
    ro, _, rq, rk, rv = ref
    assert (out.float().cpu() - ro).abs().max().item() <= OUT_TOL
    errs = [_relnorm(a, b) for a, b in ((dq, rq), (dk, rk), (dv, rv))]
    assert max(errs) <= GRAD_TOL, f"rel-norm dq/dk/dv = {errs}"


def test_sliding_window_dense():
    import ring_swa

    q, k, v, do = _rand((2, 500, 8, 128), 1), _rand((2, 500, 2, 128), 2), _rand((2, 500, 2, 128), 3), \
        _rand((2, 500, 8, 128), 4)
    ref = O.attention_fwd_bwd(lambda q, k, v: O.sliding_window_attn(q, k, v, 100), q, k, v, do)
    _compare(_gpu_fwd_bwd(lambda q, k, v: ring_swa.ring_sliding_window_attn(q, k, v, 100), q, k, v, do), ref)


def test_cpu_plumbing_shape_in_16_bits():
    """The shape of the CPU-runnable configuration -- batch 1, seq 1024, 4 q = 4 kv heads,
    head_dim 64, window 256, seed 0, scale 1/8, dO ~ N(0,1): the workload the CPU baseline of
    the benchmark times in fp32 -- through the HIP kernels in bf16 and fp16, against the fp32
    oracle on the same (rounded) inputs."""
    import ring_swa

    torch.manual_seed(0)
    q32, k32, v32, do32 = (torch.randn(1, 1024, 4, 64) for _ in range(4))
    for dtype in (torch.bfloat16, torch.float16):
        q, k, v, do = (t.to(dtype) for t in (q32, k32, v32, do32))
        ref = O.attention_fwd_bwd(lambda q, k, v: O.sliding_window_attn(q, k, v, 256, 1 / 8), q, k, v, do)
        fn = lambda q, k, v: ring_swa.ring_sliding_window_attn(q, k, v, 256, softmax_scale=1 / 8)  # noqa: E731
        _compare(_gpu_fwd_bwd(fn, q, k, v, do), ref)


def test_sliding_window_varlen_positional_like_upstream_callers():
    import ring_swa

    lens = [300, 64, 449, 7]
    cu = torch.tensor([0] + list(itertools.accumulate(lens)), dtype=torch.int32)
    t = int(cu[-1])
    q, k, v, do = _rand((t, 8, 128), 1), _rand((t, 2, 128), 2), _rand((t, 2, 128), 3), _rand((t, 8, 128), 4)
    ref = O.attention_fwd_bwd(lambda q, k, v: O.sliding_window_attn_varlen(q, k, v, 128, cu), q, k, v, do)
    dcu = cu.cuda()
    # positional through cp_next_global_rank, as test/test_ring_swa_varlen.py calls it
    fn = lambda q, k, v: ring_swa.ring_sliding_window_attn_varlen(q, k, v, 128, dcu, None, 1, 0, 0, 0)
    _compare(_gpu_fwd_bwd(fn, q, k, v, do), ref)


@pytest.mark.parametrize("impl", ["fused", "split"])
@pytest.mark.parametrize("n_sink,w", [(1, 128), (4, 60), (4, 1000)])
def test_streaming_llm_dense(impl, n_sink, w):
    import ring_swa

    s = 640
    q, k, v, do = _rand((2, s, 8, 64), 1), _rand((2, s, 2, 64), 2), _rand((2, s, 2, 64), 3), _rand((2, s, 8, 64), 4)
    k[:, :n_sink] *= 4  # peaked mass on the sinks
    ref = O.attention_fwd_bwd(lambda q, k, v: O.streaming_llm_attn(q, k, v, w, n_sink=n_sink), q, k, v, do)
    fn = lambda q, k, v: ring_swa.ring_streaming_llm_attn(q, k, v, w, num_sink_tokens=n_sink, impl=impl)
    _compare(_gpu_fwd_bwd(fn, q, k, v, do), ref)
    if n_sink == 1:
        # the reference's own composition (window over tokens 1.., sink, pad, merge)
        ro, _ = O.streaming_llm_split_reference(q, k, v, w)
        out = fn(q.cuda(), k.cuda(), v.cuda())
        assert (out.float().cpu() - ro).abs().max().item() <= OUT_TOL


@pytest.mark.parametrize("impl", ["fused", "split"])
@pytest.mark.parametrize("n_sink", [1, 4])
def test_streaming_llm_varlen(impl, n_sink):
    import ring_swa

    lens = [700, 2, 300, 130]  # one sequence shorter than the sink count
    cu = torch.tensor([0] + list(itertools.accumulate(lens)), dtype=torch.int32)
    t, w = int(cu[-1]), 100
    q, k, v, do = _rand((t, 8, 128), 1), _rand((t, 2, 128), 2), _rand((t, 2, 128), 3), _rand((t, 8, 128), 4)
    # every sequence starts with the same tokens (the precondition of the upstream packed
    # path, test/test_ring_slm_varlen.py:145-147), sink keys scaled x4
    k[:n_sink] *= 4
    for b in range(1, len(lens)):
        n = min(n_sink, lens[b])
        for t_ in (q, k, v):
            t_[cu[b]:cu[b] + n] = t_[:n]
    ref = O.attention_fwd_bwd(
        lambda q, k, v: O.streaming_llm_attn_varlen(q, k, v, w, cu, n_sink=n_sink), q, k, v, do)
    dcu = cu.cuda()
    fn = lambda q, k, v: ring_swa.ring_streaming_llm_attn_varlen(
        q, k, v, w, dcu, cp_size=1, num_sink_tokens=n_sink, impl=impl)
    _compare(_gpu_fwd_bwd(fn, q, k, v, do), ref)


@pytest.mark.parametrize("w,cp", [(300, 4), (256, 2), (700, 4), (1100, 4)])
@pytest.mark.parametrize("ring_dtypes", [False, True])
def test_rank_shares_concatenate_to_the_global_result(w, cp, ring_dtypes):
    """Every virtual rank gets its chunk + the chunks before it; outputs and gradients,
    put back together, must equal the single-GPU call on the whole sequence."""
    import ring_swa
    from ring_swa.rank_share import ring_comm_times

    s_loc, hq, hk, d = 256, 4, 2, 128
    total = s_loc * cp
    q, k, v, do = _rand((1, total, hq, d), 1), _rand((1, total, hk, d), 2), _rand((1, total, hk, d), 3), \
        _rand((1, total, hq, d), 4)
    ref = O.attention_fwd_bwd(lambda q, k, v: O.sliding_window_attn(q, k, v, w), q, k, v, do)
    hops = ring_comm_times(w, s_loc, cp)
    outs, dqs = [], []
    dk = torch.zeros(1, total, hk, d)
    dv = torch.zeros(1, total, hk, d)
    for r in range(cp):
        sl = slice(r * s_loc, (r + 1) * s_loc)
        qr, kr, vr = (t[:, sl].cuda().requires_grad_() for t in (q, k, v))
        prev = []
        for i in range(1, hops + 1):
            if r - i >= 0:
                ps = slice((r - i) * s_loc, (r - i + 1) * s_loc)
                prev.append(torch.stack([k[:, ps], v[:, ps]]).cuda().requires_grad_())
        out = ring_swa.ring_rank_share_attn(qr, kr, vr, prev, w, cp, r, ring_dtypes=ring_dtypes)
        out.backward(do[:, sl].cuda())
        outs.append(out.detach().float().cpu())
        dqs.append(qr.grad.float().cpu())
        dk[:, sl] += kr.grad.float().cpu()
        dv[:, sl] += vr.grad.float().cpu()
        for i, p in enumerate(prev, start=1):
            ps = slice((r - i) * s_loc, (r - i + 1) * s_loc)
            dk[:, ps] += p.grad[0].float().cpu()
            dv[:, ps] += p.grad[1].float().cpu()
    torch.cuda.synchronize()
    _compare((torch.cat(outs, 1), torch.cat(dqs, 1), dk, dv), ref)
    # and against this build's own single-call kernel path (the reference's invariant)
    glob = ring_swa.ring_sliding_window_attn(q.cuda(), k.cuda(), v.cuda(), w).float().cpu()
    assert (torch.cat(outs, 1) - glob).abs().max().item() <= OUT_TOL


@pytest.mark.parametrize("w,s_loc,batch", [(300, 512, 1), (512, 512, 2), (100, 768, 1)])
def test_two_block_step_is_the_same_bits_with_16_bit_and_with_fp32_accumulators(w, s_loc, batch):
    """A step of two blocks (window no longer than a chunk): the 16-bit route (second block
    merged in its forward epilogue, dq summed inside the own-chunk dQ kernel) and the route
    through the fp32 / fp64 / fp32 accumulators of ring_swa/sliding_window/nonvarlen.py:53-59,
    203-206 both make one fp32 combination of the two blocks' 16-bit results and round once."""
    import ring_swa

    hq, hk, d, cp, rank = 8, 2, 128, 4, 2
    q, do = _rand((batch, s_loc, hq, d), 11), _rand((batch, s_loc, hq, d), 12)
    k, v = _rand((batch, s_loc, hk, d), 13), _rand((batch, s_loc, hk, d), 14)
    prev = _rand((2, batch, s_loc, hk, d), 15)
    got = {}
    for route, kw in (("narrow", {"one_pass": False}), ("wide", {"ring_dtypes": True})):
        qg, kg, vg, pg = (t.cuda().requires_grad_() for t in (q, k, v, prev))
        out = ring_swa.ring_rank_share_attn(qg, kg, vg, [pg], w, cp, rank, **kw)
        out.backward(do.cuda())
        got[route] = (out.detach(), qg.grad, kg.grad, vg.grad, pg.grad)
    for a, b in zip(got["narrow"], got["wide"]):
        assert a.dtype == b.dtype and torch.equal(a, b)


@pytest.mark.parametrize("w", [200, 600])
def test_rank_shares_varlen_concatenate_to_the_global_result(w):
    import ring_swa
    from ring_swa.rank_share import ring_comm_times

    cp, s_loc, hq, hk, d = 4, 256, 4, 2, 128
    total = cp * s_loc
    lens = [100, 500, 30, 394]  # boundaries fall inside chunks; a sequence spans 3 ranks
    assert sum(lens) == total
    cu = [0] + list(itertools.accumulate(lens))
    q, k, v, do = _rand((total, hq, d), 1), _rand((total, hk, d), 2), _rand((total, hk, d), 3), \
        _rand((total, hq, d), 4)
    ref = O.attention_fwd_bwd(lambda q, k, v: O.sliding_window_attn_varlen(q, k, v, w, cu), q, k, v, do)
    hops = ring_comm_times(w, s_loc, cp)
    outs, dqs = [], []
    dk, dv = torch.zeros(total, hk, d), torch.zeros(total, hk, d)
    for r in range(cp):
        sl = slice(r * s_loc, (r + 1) * s_loc)
        qr, kr, vr = (t[sl].cuda().requires_grad_() for t in (q, k, v))
        prev = []
        for i in range(1, hops + 1):
            if r - i >= 0:
                ps = slice((r - i) * s_loc, (r - i + 1) * s_loc)
                prev.append(torch.stack([k[ps], v[ps]]).cuda().requires_grad_())
        out = ring_swa.ring_rank_share_attn_varlen(qr, kr, vr, prev, w, cu, cp, r)
        out.backward(do[sl].cuda())
        outs.append(out.detach().float().cpu())
        dqs.append(qr.grad.float().cpu())
        dk[sl] += kr.grad.float().cpu()
        dv[sl] += vr.grad.float().cpu()
        for i, p in enumerate(prev, start=1):
            ps = slice((r - i) * s_loc, (r - i + 1) * s_loc)
            dk[ps] += p.grad[0].float().cpu()
            dv[ps] += p.grad[1].float().cpu()
    torch.cuda.synchronize()
    _compare((torch.cat(outs, 0), torch.cat(dqs, 0), dk, dv), ref)
