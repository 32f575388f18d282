"""Pins for the CPU oracle: every oracle function is checked against something
it does not itself compute — a library routine, a closed form, a brute-force
loop, ``gradcheck`` or an algebraic invariant — chosen so that a dropped term,
a wrong sign/index or a transposed operand fails at least one check.
"""
import itertools
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import attention_oracle as O

torch.manual_seed(1234)


def rnd(*shape, dtype=torch.float64):
    return torch.randn(*shape, dtype=dtype)


# ------------------------------------------------------------------ masks
@pytest.mark.parametrize("sq,sk", [(5, 5), (3, 7), (7, 3), (1, 4), (6, 1)])
@pytest.mark.parametrize("window", [(-1, -1), (2, 0), (0, 0), (1, 2), (-1, 0), (3, -1), (0, 6)])
@pytest.mark.parametrize("causal", [False, True])
def test_window_allowed_bruteforce(sq, sk, window, causal):
    """flash-attn rule stated with loops: key j visible from row i iff
    i + sk - sq - left <= j <= i + sk - sq + right (causal => right = 0)."""
    got = O.window_allowed(sq, sk, window, causal)
    wl, wr = window
    if causal:
        wr = 0
    for i in range(sq):
        for j in range(sk):
            lo = i + sk - sq - wl if wl >= 0 else -10**9
            hi = i + sk - sq + wr if wr >= 0 else 10**9
            assert bool(got[i, j]) == (lo <= j <= hi), (i, j)


def test_sink_mask_matches_band_or_column():
    """One sink == the band mask with column 0 forced on, made causal
    (test/test_local_slm.py:58-63 builds it exactly so for sq == sk)."""
    s, w = 9, 3
    got = O.window_allowed(s, s, (w, 0), True, n_sink=1)
    band = O.window_allowed(s, s, (w, 0), True)
    want = band.clone()
    want[:, 0] = True
    assert torch.equal(got, want)
    got4 = O.window_allowed(s, s, (w, 0), True, n_sink=4)
    for i in range(s):
        for j in range(s):
            assert bool(got4[i, j]) == (j <= i and (i - j <= w or j < 4))


# ------------------------------------------------------------------ forward
def test_full_window_equals_sdpa():
    q, k, v = rnd(2, 6, 4, 8), rnd(2, 9, 4, 8), rnd(2, 9, 4, 8)
    out, lse = O.window_attention(q, k, v, None, (-1, -1), False, compute_dtype=torch.float64)
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2))
    torch.testing.assert_close(out, ref.transpose(1, 2), atol=1e-12, rtol=1e-10)


def test_wide_causal_window_equals_sdpa_causal_and_gqa():
    s = 11
    q, k, v = rnd(1, s, 6, 8), rnd(1, s, 2, 8), rnd(1, s, 2, 8)
    out, _ = O.sliding_window_attn(q, k, v, window_size=s - 1, compute_dtype=torch.float64)
    kk = k.repeat_interleave(3, dim=2)
    vv = v.repeat_interleave(3, dim=2)
    ref = F.scaled_dot_product_attention(
        q.transpose(1, 2), kk.transpose(1, 2), vv.transpose(1, 2), is_causal=True
    )
    torch.testing.assert_close(out, ref.transpose(1, 2), atol=1e-12, rtol=1e-10)
    # GQA mapping is h // group, not h % group: head 1 must use kv head 0
    out1, _ = O.sliding_window_attn(q[:, :, 1:2], k[:, :, 0:1], v[:, :, 0:1], s - 1,
                                    compute_dtype=torch.float64)
    torch.testing.assert_close(out[:, :, 1:2], out1, atol=1e-12, rtol=1e-10)


def test_window_zero_returns_own_value_and_score():
    s = 7
    q, k, v = rnd(2, s, 4, 8), rnd(2, s, 2, 8), rnd(2, s, 2, 8)
    scale = 0.37
    out, lse = O.sliding_window_attn(q, k, v, 0, softmax_scale=scale, compute_dtype=torch.float64)
    torch.testing.assert_close(out, v.repeat_interleave(2, dim=2), atol=1e-12, rtol=0)
    want = scale * (q * k.repeat_interleave(2, dim=2)).sum(-1).transpose(1, 2)
    torch.testing.assert_close(lse, want, atol=1e-12, rtol=0)


def test_bruteforce_loops_out_and_lse():
    b, sq, sk, hq, hk, d = 1, 4, 6, 2, 1, 3
    q, k, v = rnd(b, sq, hq, d), rnd(b, sk, hk, d), rnd(b, sk, hk, d)
    window, scale = (2, 1), 0.5
    out, lse = O.window_attention(q, k, v, scale, window, False, compute_dtype=torch.float64)
    for h in range(hq):
        for i in range(sq):
            ws, acc = [], [0.0] * d
            for j in range(sk):
                if i + sk - sq - 2 <= j <= i + sk - sq + 1:
                    sc = scale * sum(float(q[0, i, h, c]) * float(k[0, j, 0, c]) for c in range(d))
                    ws.append((math.exp(sc), j))
            z = sum(w for w, _ in ws)
            for w, j in ws:
                for c in range(d):
                    acc[c] += w / z * float(v[0, j, 0, c])
            assert abs(float(lse[0, h, i]) - math.log(z)) < 1e-12
            for c in range(d):
                assert abs(float(out[0, i, h, c]) - acc[c]) < 1e-12


def test_empty_rows_are_merge_identity():
    # sq > sk with causal bottom-right alignment: the first sq - sk rows see nothing
    q, k, v = rnd(1, 6, 2, 4), rnd(1, 3, 2, 4), rnd(1, 3, 2, 4)
    out, lse = O.window_attention(q, k, v, None, (-1, 0), True, compute_dtype=torch.float64)
    assert torch.all(out[:, :3] == 0) and torch.all(torch.isinf(lse[:, :, :3]) & (lse[:, :, :3] < 0))
    assert torch.isfinite(lse[:, :, 3:]).all()


def test_varlen_equals_concat_of_dense():
    lens = [3, 1, 5, 2]
    cu = [0] + list(itertools.accumulate(lens))
    t = cu[-1]
    q, k, v = rnd(t, 4, 8), rnd(t, 2, 8), rnd(t, 2, 8)
    out, lse = O.sliding_window_attn_varlen(q, k, v, 2, cu, compute_dtype=torch.float64)
    assert out.shape == (t, 4, 8) and lse.shape == (4, t)
    for b, L in enumerate(lens):
        sl = slice(cu[b], cu[b + 1])
        o1, l1 = O.sliding_window_attn(q[sl][None], k[sl][None], v[sl][None], 2,
                                       compute_dtype=torch.float64)
        torch.testing.assert_close(out[sl], o1[0], atol=1e-12, rtol=0)
        torch.testing.assert_close(lse[:, sl], l1[0], atol=1e-12, rtol=0)
    # a token never sees another sequence: perturbing sequence 0 leaves the rest untouched
    k2 = k.clone()
    k2[:3] += 1.0
    out2, _ = O.sliding_window_attn_varlen(q, k2, v, 2, cu, compute_dtype=torch.float64)
    assert torch.equal(out2[3:], out[3:]) and not torch.equal(out2[:3], out[:3])


# ------------------------------------------------------------------ streaming-LLM
@pytest.mark.parametrize("w", [0, 1, 3, 20])
def test_slm_reference_composition_equals_closed_form(w):
    s = 10
    q, k, v = rnd(2, s, 4, 8), rnd(2, s, 2, 8), rnd(2, s, 2, 8)
    o1, l1 = O.streaming_llm_attn(q, k, v, w, compute_dtype=torch.float64)
    o2, l2 = O.streaming_llm_split_reference(q, k, v, w, compute_dtype=torch.float64)
    torch.testing.assert_close(o1, o2, atol=1e-12, rtol=1e-10)
    torch.testing.assert_close(l1, l2, atol=1e-12, rtol=1e-10)
    if w >= s:
        oc, lc = O.sliding_window_attn(q, k, v, s, compute_dtype=torch.float64)
        torch.testing.assert_close(o1, oc, atol=1e-12, rtol=1e-10)


def test_slm_varlen_per_sequence_sink():
    lens = [4, 6]
    cu = [0, 4, 10]
    q, k, v = rnd(10, 2, 4), rnd(10, 2, 4), rnd(10, 2, 4)
    out, lse = O.streaming_llm_attn_varlen(q, k, v, 1, cu, n_sink=2, compute_dtype=torch.float64)
    for b in range(2):
        sl = slice(cu[b], cu[b + 1])
        o1, l1 = O.streaming_llm_attn(q[sl][None], k[sl][None], v[sl][None], 1, n_sink=2,
                                      compute_dtype=torch.float64)
        torch.testing.assert_close(out[sl], o1[0], atol=1e-12, rtol=0)


# ------------------------------------------------------------------ merge
def _partials(sq=6, sk=10, hq=4, hk=2, d=8):
    q, k, v = rnd(2, sq, hq, d), rnd(2, sk, hk, d), rnd(2, sk, hk, d)
    return q, k, v


def test_merge_split_kv_invariance():
    """attention over A u B == merge(attention(A), attention(B)): pins the LSE
    (natural log, not log2; per row; [B,H,S] layout) and the merge weights."""
    q, k, v = _partials()
    full_o, full_l = O.window_attention(q, k, v, compute_dtype=torch.float64)
    oa, la = O.window_attention(q, k[:, :4], v[:, :4], compute_dtype=torch.float64)
    ob, lb = O.window_attention(q, k[:, 4:], v[:, 4:], compute_dtype=torch.float64)
    om, lm = O.merge(oa, la, ob, lb)
    torch.testing.assert_close(om, full_o, atol=1e-12, rtol=1e-10)
    torch.testing.assert_close(lm, full_l, atol=1e-12, rtol=1e-10)
    torch.testing.assert_close(lm, torch.logaddexp(la, lb), atol=1e-12, rtol=1e-12)


def test_merge_commutative_identity_and_forms_agree():
    q, k, v = _partials()
    oa, la = O.window_attention(q, k[:, :4], v[:, :4], compute_dtype=torch.float64)
    ob, lb = O.window_attention(q, k[:, 4:], v[:, 4:], compute_dtype=torch.float64)
    o1, l1 = O.merge(oa, la, ob, lb)
    o2, l2 = O.merge(ob, lb, oa, la)
    torch.testing.assert_close(o1, o2, atol=1e-13, rtol=0)
    torch.testing.assert_close(l1, l2, atol=1e-13, rtol=0)
    zero, ninf = torch.zeros_like(oa), torch.full_like(la, O.NEG_INF)
    o3, l3 = O.merge(zero, ninf, oa, la)
    assert torch.equal(o3, oa) and torch.equal(l3, la)
    o4, l4 = O.merge(oa, la, zero, ninf)
    assert torch.equal(o4, oa) and torch.equal(l4, la)
    o5, l5 = O.merge(zero, ninf, zero, ninf)
    assert torch.all(o5 == 0) and torch.all(torch.isinf(l5) & (l5 < 0))
    o6, l6 = O.merge_softplus(oa, la, ob, lb)
    torch.testing.assert_close(o1, o6, atol=1e-12, rtol=1e-10)
    torch.testing.assert_close(l1, l6, atol=1e-12, rtol=1e-10)


def test_merge_mixed_dtypes_follow_accumulator():
    """Ring dtypes (ring_swa/sliding_window/nonvarlen.py:53-59): fp32 o, fp64 lse,
    bf16 new o, fp32 new lse -> result keeps the accumulator dtypes."""
    q, k, v = _partials()
    oa, la = O.window_attention(q, k[:, :4], v[:, :4], compute_dtype=torch.float64)
    ob, lb = O.window_attention(q, k[:, 4:], v[:, 4:], compute_dtype=torch.float64)
    om, lm = O.merge(oa.float(), la, ob.bfloat16(), lb.float())
    assert om.dtype == torch.float32 and lm.dtype == torch.float64
    ref_o, ref_l = O.merge(oa, la, ob, lb)
    torch.testing.assert_close(om.double(), ref_o, atol=2e-2, rtol=0)
    torch.testing.assert_close(lm, ref_l, atol=1e-5, rtol=0)


# ------------------------------------------------------------------ backward
def test_gradcheck_masked_attention():
    q = rnd(1, 4, 2, 3).requires_grad_()
    k = rnd(1, 5, 1, 3).requires_grad_()
    v = rnd(1, 5, 1, 3).requires_grad_()
    allowed = O.window_allowed(4, 5, (2, 1), False)

    def f(q, k, v):
        o, l = O.masked_attention(q, k, v, allowed, 0.7, torch.float64)
        return o, l

    assert torch.autograd.gradcheck(f, (q, k, v), eps=1e-6, atol=1e-6)


def test_bwd_from_stats_equals_autograd_and_sums_over_blocks():
    """sum over KV blocks of bwd(block; o_final, lse_final) == autograd of the
    global attention: the 'merge backward' contract of the ring."""
    b, s, hq, hk, d, w = 2, 12, 4, 2, 8, 5
    q, k, v, do = rnd(b, s, hq, d), rnd(b, s, hk, d), rnd(b, s, hk, d), rnd(b, s, hq, d)
    out, lse, dq, dk, dv = O.attention_fwd_bwd(
        lambda q, k, v: O.sliding_window_attn(q, k, v, w, compute_dtype=torch.float64), q, k, v, do
    )
    allowed = O.window_allowed(s, s, (w, 0), True)
    g = O.attention_bwd_from_stats(q, k, v, out, lse, do, allowed, compute_dtype=torch.float64)
    for a, r in zip(g, (dq, dk, dv)):
        torch.testing.assert_close(a, r, atol=1e-11, rtol=1e-9)
    # split keys into two blocks, each with its restriction of the mask
    dq2 = torch.zeros_like(dq)
    dk2 = torch.zeros_like(dk)
    dv2 = torch.zeros_like(dv)
    for sl in (slice(0, 7), slice(7, s)):
        a, bb, c = O.attention_bwd_from_stats(q, k[:, sl], v[:, sl], out, lse, do, allowed[:, sl],
                                              compute_dtype=torch.float64)
        dq2 += a
        dk2[:, sl] += bb
        dv2[:, sl] += c
    for a, r in zip((dq2, dk2, dv2), (dq, dk, dv)):
        torch.testing.assert_close(a, r, atol=1e-11, rtol=1e-9)


# ------------------------------------------------------------------ ring geometry
def _global_mask(total, w, cu=None):
    pos = torch.arange(total)
    if cu is None:
        sid = torch.zeros(total, dtype=torch.long)
    else:
        sid = torch.bucketize(pos, torch.tensor(cu[1:]), right=True)
    return O.global_band_allowed(pos, pos, sid, sid, w)


@pytest.mark.parametrize("seq_len", [4, 5])
@pytest.mark.parametrize("cp", [2, 3, 4])
def test_ring_steps_nonvarlen_tile_the_global_band(seq_len, cp):
    total = seq_len * cp
    for w in range(1, total + 2):
        want = _global_mask(total, w)
        for r in range(cp):
            got = torch.zeros(seq_len, total, dtype=torch.bool)
            steps = O.ring_steps_nonvarlen(seq_len, w, cp, r)
            for (i, qs, ks, window, causal) in steps:
                kv0 = (r - i) * seq_len
                sq = qs.stop - qs.start
                sk = ks.stop - ks.start
                m = O.window_allowed(sq, sk, window, causal)
                blk = got[qs, kv0 + ks.start: kv0 + ks.stop]
                assert not (blk & m).any(), "blocks overlap"
                got[qs, kv0 + ks.start: kv0 + ks.stop] = blk | m
            assert torch.equal(got, want[r * seq_len:(r + 1) * seq_len]), (w, r)


def test_ring_steps_varlen_tile_the_global_band():
    g = torch.Generator().manual_seed(7)
    for trial in range(60):
        cp = int(torch.randint(2, 5, (1,), generator=g))
        seq_len = int(torch.randint(3, 7, (1,), generator=g))
        total = cp * seq_len
        cuts = sorted(set(torch.randint(1, total, (int(torch.randint(0, 4, (1,), generator=g)),),
                                        generator=g).tolist()))
        cu = [0] + cuts + [total]
        w = int(torch.randint(1, total + 1, (1,), generator=g))
        want = _global_mask(total, w, cu)
        for r in range(cp):
            local_cu, steps = O.ring_steps_varlen(cu, seq_len, w, cp, r)
            got = torch.zeros(seq_len, total, dtype=torch.bool)
            for (i, qs, ks, window, causal) in steps:
                kv0 = (r - i) * seq_len
                if i == 0:
                    for a, b in zip(local_cu[:-1], local_cu[1:]):
                        m = O.window_allowed(b - a, b - a, window, causal)
                        got[a:b, kv0 + a: kv0 + b] |= m
                else:
                    m = O.window_allowed(qs.stop - qs.start, ks.stop - ks.start, window, causal)
                    got[qs, kv0 + ks.start: kv0 + ks.stop] |= m
            assert torch.equal(got, want[r * seq_len:(r + 1) * seq_len]), (cu, seq_len, w, r)


# ------------------------------------------------------------------ counters
def test_pair_counters_match_masks():
    for L in (1, 5, 17):
        for w in (0, 3, 16, 40):
            assert O.band_pairs(L, w) == int(O.window_allowed(L, L, (w, 0), True).sum())
            for n in (1, 4):
                tot = int(O.window_allowed(L, L, (w, 0), True, n_sink=n).sum())
                assert O.band_pairs(L, w) + O.sink_extra_pairs(L, w, n) == tot
    # figures quoted for the benchmark shapes
    assert O.band_pairs(8192, 1000) == 7_699_692
    assert O.band_pairs(1024, 256) == 230_272
    assert O.band_pairs(8192, 4096) + 4096 * 4097 // 2 == 33_562_624 == 8192 * 4097


def test_flop_counter_reproduces_the_quoted_workloads():
    """4 / 10 / 14 x D x pairs x heads x batch against the totals quoted for the benchmark
    shapes (0.2523 / 0.6308 / 0.8831 TFLOP for batch 2, 8192 tokens, 32 heads, window 1000;
    0.5499 / 1.3747 / 1.9246 TFLOP for the rank share; 0.83 GFLOP for the CPU case) and
    against a direct count on a small mask."""
    f, b, t = O.attention_flops(O.band_pairs(8192, 1000), 128, 32, 2)
    assert (round(f / 1e12, 4), round(b / 1e12, 4), round(t / 1e12, 4)) == (0.2523, 0.6308, 0.8831)
    f, b, t = O.attention_flops(8192 * 4097, 128, 32)
    assert (round(f / 1e12, 4), round(b / 1e12, 4), round(t / 1e12, 4)) == (0.5499, 1.3747, 1.9246)
    assert round(O.attention_flops(O.band_pairs(1024, 256), 64, 4)[2] / 1e9, 2) == 0.83
    m = O.window_allowed(9, 9, (3, 0), True)
    # one multiply-add per (pair, d) and GEMM: forward 2 GEMMs, backward 5
    assert O.attention_flops(int(m.sum()), 16, 3, 2) == tuple(
        g * 2 * int(m.sum()) * 16 * 3 * 2 for g in (2, 5, 7))


def test_global_mask_with_sinks_equals_the_per_sequence_rule():
    """The sink branch of the global formula: per sequence it is the dense rule with sinks
    (pinned above by brute force), and no pair ever crosses a sequence boundary."""
    cu = [0, 5, 6, 17, 30]
    total = cu[-1]
    pos = torch.arange(total)
    sid = torch.bucketize(pos, torch.tensor(cu[1:]), right=True)
    start = torch.tensor(cu)[sid]
    for w in (0, 2, 7, 40):
        for n in (1, 4):
            got = O.global_band_allowed(pos, pos, sid, sid, w, n_sink=n, seq_start_k=start)
            want = torch.zeros(total, total, dtype=torch.bool)
            for a, b in zip(cu[:-1], cu[1:]):
                want[a:b, a:b] = O.window_allowed(b - a, b - a, (w, 0), True, n_sink=n)
            assert torch.equal(got, want), (w, n)
            # brute force of the stated rule
            for p in range(total):
                for t in range(total):
                    rule = sid[p] == sid[t] and t <= p and (p - t <= w or t - cu[sid[t]] < n)
                    assert bool(got[p, t]) == bool(rule)


def test_explicit_shift_of_the_window_rule_by_brute_force():
    """``shift`` moves the diagonal: key j visible from row i iff j <= i + shift + right and
    j >= i + shift - left (negative bound: none); the default is ``sk - sq``."""
    for sq, sk, window, shift in ((7, 3, (-1, 0), -4), (5, 9, (2, 1), 0), (6, 6, (1, -1), 3),
                                  (4, 2, (-1, 0), -9), (8, 8, (3, 0), None)):
        got = O.window_allowed(sq, sk, window, False, shift=shift)
        sh = sk - sq if shift is None else shift
        for i in range(sq):
            for j in range(sk):
                want = True
                if window[1] >= 0:
                    want &= j <= i + sh + window[1]
                if window[0] >= 0:
                    want &= j >= i + sh - window[0]
                assert bool(got[i, j]) == want, (sq, sk, window, shift, i, j)
