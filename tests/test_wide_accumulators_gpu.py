"""The ring loops' accumulators taken by the kernels as they are (``wide`` of the C ABI): fp32
running output with fp64 running LSE in the forward, fp32 ``dq`` / ``dk`` / ``dv`` in the backward
(``ring_swa/sliding_window/nonvarlen.py:53-59, 203-206, 318-321``).  Everything here is bit
equality with the unfused flow on the same inputs: a forward into 16-bit temporaries followed by
``rswa_merge_attn_out`` on the accumulators, and 16-bit gradients added to fp32 buffers."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _rand(shape, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g).to(dtype).cuda()


CASES = [
    # (B, Sq, Sk, Hq, Hkv, D, window, causal, dtype)
    (2, 300, 300, 8, 2, 128, (100, 0), True, torch.bfloat16),
    (1, 513, 700, 4, 4, 64, (64, 0), True, torch.float16),
    (1, 200, 456, 6, 2, 128, (0, 456), False, torch.bfloat16),   # a corner block of the ring
    (1, 333, 200, 4, 2, 128, (40, 0), True, torch.bfloat16),     # leading rows see nothing
    (1, 2048, 40000, 2, 2, 128, (4000, 0), True, torch.bfloat16),  # 157 key tiles x 2 heads: no split
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "x".join(str(x) for x in c[:8]))
def test_forward_into_and_onto_the_ring_accumulators(case):
    from ring_swa.ops import attn_fwd, merge_attn_out

    b, sq, sk, hq, hk, d, window, causal, dtype = case
    q, k, v = _rand((b, sq, hq, d), 1, dtype), _rand((b, sk, hk, d), 2, dtype), _rand((b, sk, hk, d), 3, dtype)
    k2, v2 = _rand((b, sk, hk, d), 5, dtype), _rand((b, sk, hk, d), 6, dtype)
    out16, lse32 = attn_fwd(q, k, v, None, window, causal)
    # written as accumulators: the 16-bit values, exactly
    acc = torch.full(q.shape, float("nan"), dtype=torch.float32, device="cuda")
    lacc = torch.full(lse32.shape, float("nan"), dtype=torch.float64, device="cuda")
    got = attn_fwd(q, k, v, None, window, causal, into=(acc, lacc))
    assert got[0] is acc and got[1] is lacc
    assert torch.equal(acc, out16.float()) and torch.equal(lacc, lse32.double())
    # a second block merged into them == 16-bit temporaries + the merge kernel
    ref_o, ref_l = acc.clone(), lacc.clone()
    t_o, t_l = attn_fwd(q, k2, v2, None, window, causal)
    merge_attn_out(ref_o, ref_l, t_o, t_l)
    attn_fwd(q, k2, v2, None, window, causal, accumulate_into=(acc, lacc))
    assert torch.equal(acc, ref_o) and torch.equal(lacc, ref_l)
    # from the merge identity (zeros, -inf), on a sliced view of larger accumulators
    big_o = torch.zeros(b, sq + 7, hq, d, dtype=torch.float32, device="cuda")
    big_l = torch.full((b, hq, sq + 7), float("-inf"), dtype=torch.float64, device="cuda")
    attn_fwd(q, k, v, None, window, causal, accumulate_into=(big_o[:, 3:3 + sq], big_l[:, :, 3:3 + sq]))
    assert torch.equal(big_o[:, 3:3 + sq], out16.float())
    assert torch.equal(big_l[:, :, 3:3 + sq], lse32.double())
    assert big_o[:, :3].abs().max() == 0 and big_o[:, 3 + sq:].abs().max() == 0


@pytest.mark.parametrize("case", CASES, ids=lambda c: "x".join(str(x) for x in c[:8]))
def test_backward_into_and_onto_fp32_gradient_accumulators(case):
    from ring_swa.ops import attn_bwd, attn_fwd

    b, sq, sk, hq, hk, d, window, causal, dtype = case
    q, k, v = _rand((b, sq, hq, d), 1, dtype), _rand((b, sk, hk, d), 2, dtype), _rand((b, sk, hk, d), 3, dtype)
    do = _rand((b, sq, hq, d), 4, dtype)
    out, lse = attn_fwd(q, k, v, None, window, causal)
    gq, gk, gv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    attn_bwd(q, k, v, out, lse, do, gq, gk, gv, None, window, causal)
    nan32 = lambda t: torch.full(t.shape, float("nan"), dtype=torch.float32, device="cuda")  # noqa: E731
    # written as fp32: the 16-bit gradients, exactly
    wq, wk, wv = nan32(q), nan32(k), nan32(v)
    attn_bwd(q, k, v, out, lse, do, wq, wk, wv, None, window, causal)
    assert torch.equal(wq, gq.float()) and torch.equal(wk, gk.float()) and torch.equal(wv, gv.float())
    # added to what the accumulators hold
    iq, ik, iv = (_rand(t.shape, 7 + i, torch.float32) for i, t in enumerate((q, k, v)))
    aq, ak, av = iq.clone(), ik.clone(), iv.clone()
    attn_bwd(q, k, v, out, lse, do, aq, ak, av, None, window, causal, dq_accumulate=True,
             dkv_accumulate=True)
    assert torch.equal(aq, iq + gq.float())
    assert torch.equal(ak, ik + gk.float()) and torch.equal(av, iv + gv.float())
    # mixed: fp32 dq accumulated, 16-bit dk / dv (what a ring sends back to the keys' owner)
    aq, mk, mv = iq.clone(), torch.empty_like(k), torch.empty_like(v)
    attn_bwd(q, k, v, out, lse, do, aq, mk, mv, None, window, causal, dq_accumulate=True)
    assert torch.equal(aq, iq + gq.float()) and torch.equal(mk, gk) and torch.equal(mv, gv)
    # the dS hand-off route writes dq through the same epilogue
    hq_, hk_, hv_ = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    attn_bwd(q, k, v, out, lse, do, hq_, hk_, hv_, None, window, causal, handoff="force")
    aq, ak, av = iq.clone(), ik.clone(), iv.clone()
    attn_bwd(q, k, v, out, lse, do, aq, ak, av, None, window, causal, dq_accumulate=True,
             dkv_accumulate=True, handoff="force")
    assert torch.equal(aq, iq + hq_.float())
    assert torch.equal(ak, ik + hk_.float()) and torch.equal(av, iv + hv_.float())


def test_packed_and_two_key_ranges_with_fp32_accumulators():
    from ring_swa.ops import attn_bwd, attn_fwd

    hq, hk, d, w = 8, 2, 128, 200
    cu = torch.tensor([0, 130, 131, 500, 700], dtype=torch.int32, device="cuda")
    q, do = _rand((700, hq, d), 1), _rand((700, hq, d), 4)
    k, v = _rand((700, hk, d), 2), _rand((700, hk, d), 3)
    out, lse = attn_fwd(q, k, v, None, (w, 0), True, cu, cu)
    acc = torch.zeros(700, hq, d, dtype=torch.float32, device="cuda")
    lacc = torch.full((hq, 700), float("-inf"), dtype=torch.float64, device="cuda")
    attn_fwd(q, k, v, None, (w, 0), True, cu, cu, accumulate_into=(acc, lacc))
    assert torch.equal(acc, out.float()) and torch.equal(lacc, lse.double())
    gq, gk, gv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    attn_bwd(q, k, v, out, lse, do, gq, gk, gv, None, (w, 0), True, cu, cu)
    aq, ak, av = (torch.ones(t.shape, dtype=torch.float32, device="cuda") for t in (q, k, v))
    attn_bwd(q, k, v, out, lse, do, aq, ak, av, None, (w, 0), True, cu, cu, dq_accumulate=True,
             dkv_accumulate=True)
    assert torch.equal(aq, 1 + gq.float()) and torch.equal(ak, 1 + gk.float()) and torch.equal(av, 1 + gv.float())
    # keys in two row ranges (dense): both ranges' gradients as fp32
    s, tail = 768, 512
    q, do = _rand((1, s, hq, d), 1), _rand((1, s, hq, d), 4)
    k1, v1, k2, v2 = _rand((1, tail, hk, d), 2), _rand((1, tail, hk, d), 3), _rand((1, s, hk, d), 5), \
        _rand((1, s, hk, d), 6)
    out, lse = attn_fwd(q, k1, v1, None, (400, 0), True, second=(k2, v2))
    g = [torch.empty_like(t) for t in (q, k1, v1, k2, v2)]
    attn_bwd(q, k1, v1, out, lse, do, g[0], g[1], g[2], None, (400, 0), True, second=(k2, v2, g[3], g[4]))
    a = [torch.full(t.shape, 2.0, dtype=torch.float32, device="cuda") for t in (q, k1, v1, k2, v2)]
    attn_bwd(q, k1, v1, out, lse, do, a[0], a[1], a[2], None, (400, 0), True,
             second=(k2, v2, a[3], a[4]), dq_accumulate=True, dkv_accumulate=True)
    for x, y in zip(a, g):
        assert torch.equal(x, 2 + y.float())


def test_what_the_accumulator_types_refuse():
    from ring_swa.ops import attn_bwd, attn_fwd

    q, k, v, do = (_rand((1, 600, 4, 128), i) for i in range(4))
    out, lse = attn_fwd(q, k, v, None, (50, 0), True, num_sink=2)
    f32 = lambda t: torch.zeros(t.shape, dtype=torch.float32, device="cuda")  # noqa: E731
    # sink keys under a bounded window: their rows of dk / dv are overwritten by a second kernel
    with pytest.raises(NotImplementedError):
        attn_bwd(q, k, v, out, lse, do, f32(q), f32(k), f32(v), None, (50, 0), True, num_sink=2)
    # ... fp32 dq alone is fine there
    gq, wq, gk, gv = torch.empty_like(q), f32(q), torch.empty_like(k), torch.empty_like(v)
    attn_bwd(q, k, v, out, lse, do, gq, gk, gv, None, (50, 0), True, num_sink=2)
    attn_bwd(q, k, v, out, lse, do, wq, gk, gv, None, (50, 0), True, num_sink=2)
    assert torch.equal(wq, gq.float())
    with pytest.raises(AssertionError):
        attn_bwd(q, k, v, out, lse, do, gq, gk, gv, None, (50, 0), True, dkv_accumulate=True)
    with pytest.raises(AssertionError):  # fp32 output needs the fp64 LSE beside it
        attn_fwd(q, k, v, None, (50, 0), True, into=(f32(q), lse))
