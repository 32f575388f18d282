"""The four GPU configurations of the benchmark suite at their FULL shapes.

The complete problem (all heads, all tokens) runs through the public entry points,
forward and backward.  One GQA group -- kv head 0 with the q heads that share it, whose
dK / dV depend on no other head -- is then checked against the oracle's masked softmax
evaluated in fp32 on the same inputs (on the GPU: at these sizes the oracle's score
matrices take seconds there and hours on host cores).  Tolerances are those of the path:
out max-abs 2e-2, LSE 1e-3, dQ / dK / dV relative norm 5e-2 (held to 1e-2 here).  Every other head is covered
by properties that need no reference: finite values, and run-to-run bit equality of the
(atomic-free) kernels.
"""
import itertools
import math

import pytest
import torch

from oracle import attention_oracle as O

pytestmark = pytest.mark.gpu

OUT_TOL, LSE_TOL, GRAD_TOL = 2e-2, 1e-3, 1e-2
D = 128


def _randn(shape, seed, scale=1.0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(*shape, generator=g, device="cuda") * scale).bfloat16()


def _rel(x, ref):
    x = x.float()
    assert torch.isfinite(x).all()
    return ((x - ref).norm() / ref.norm().clamp_min(1e-30)).item()


def _mismatch_fraction(x, ref, atol=2.5e-2, rtol=2.5e-2):
    """The reference's own acceptance rule (test/test_ring_swa_nonvarlen.py:196-229):
    share of elements outside atol + rtol * |ref|."""
    bad = (x.float() - ref).abs() > atol + rtol * ref.abs()
    return bad.float().mean().item()


def _check(name, out, grads, ref_out, ref_grads):
    err = (out.float() - ref_out).abs().max().item()
    assert err <= OUT_TOL, f"{name}: out max-abs {err}"
    errs = [_rel(g, r) for g, r in zip(grads, ref_grads)]
    assert max(errs) <= GRAD_TOL, f"{name}: rel-norm dq/dk/dv = {errs}"
    # secondary, in the reference's style.  The reference asks for fewer than 0.01 % of the
    # elements off on unscaled N(0,1) inputs; the output meets that everywhere, and so do
    # the gradients except with the x4 sink keys of configuration 5, where gradients are
    # several times larger and about 0.02 % of dq end up past the bound (P and dS enter the
    # MFMAs as 16-bit values); 0.05 % is asserted for gradients.
    fr = [_mismatch_fraction(a, b) for a, b in zip((out, *grads), (ref_out, *ref_grads))]
    assert fr[0] < 1e-4 and max(fr) < 5e-4, f"{name}: mismatched fraction out/dq/dk/dv = {fr}"


def test_config2_swa_batch2_seq8192_mha_window1000():
    import ring_swa
    from ring_swa.ops import wrapped_flash_attn_fwd

    b, s, h, w = 2, 8192, 32, 1000
    q, k, v, do = (_randn((b, s, h, D), i) for i in range(4))
    qg, kg, vg = (t.clone().requires_grad_() for t in (q, k, v))
    out = ring_swa.ring_sliding_window_attn(qg, kg, vg, w)
    out.backward(do)
    _, lse = wrapped_flash_attn_fwd(q, k, v, D ** -0.5, (w, 0), True)
    hs = slice(0, 2)  # MHA: every head is its own group
    ro, rl, rq, rk, rv = O.attention_fwd_bwd(
        lambda q, k, v: O.sliding_window_attn(q, k, v, w), q[:, :, hs], k[:, :, hs], v[:, :, hs],
        do[:, :, hs])
    _check("c2", out[:, :, hs], (qg.grad[:, :, hs], kg.grad[:, :, hs], vg.grad[:, :, hs]),
           ro, (rq, rk, rv))
    assert (lse[:, hs] - rl).abs().max().item() <= LSE_TOL
    for t in (out, qg.grad, kg.grad, vg.grad):
        assert torch.isfinite(t.float()).all()
    # deterministic backward: a second run gives the same bits
    q2, k2, v2 = (t.clone().requires_grad_() for t in (q, k, v))
    ring_swa.ring_sliding_window_attn(q2, k2, v2, w).backward(do)
    assert torch.equal(q2.grad, qg.grad) and torch.equal(k2.grad, kg.grad) and torch.equal(v2.grad, vg.grad)


@pytest.mark.parametrize("route", ["one_pass", "two_blocks", "ring_dtypes"])
def test_config3_rank_share_chunk8192_gqa_window4096(route):
    """The three routes of the rank step: one band over [previous chunk's tail | own chunk]
    (default); own-chunk block + previous-chunk corner block merged in 16 bits (upstream's block
    structure, ring_swa/sliding_window/nonvarlen.py:95-154); the same two blocks through the
    accumulating block operators with fp32 output / fp64 LSE (what the ring over a cp_group runs)."""
    import ring_swa

    kw = {"one_pass": {}, "two_blocks": {"one_pass": False}, "ring_dtypes": {"ring_dtypes": True}}[route]
    s, hq, hk, w, cp, rank = 8192, 32, 8, 4096, 8, 1
    q, do = _randn((1, s, hq, D), 0), _randn((1, s, hq, D), 1)
    k, v = _randn((1, s, hk, D), 2), _randn((1, s, hk, D), 3)
    prev = _randn((2, 1, s, hk, D), 4)
    qg, kg, vg, pg = (t.clone().requires_grad_() for t in (q, k, v, prev))
    out = ring_swa.ring_rank_share_attn(qg, kg, vg, [pg], w, cp, rank, **kw)
    out.backward(do)
    # the same rows in the global picture: keys = previous chunk then own chunk,
    # queries aligned bottom-right, one causal band of width w
    gq, gk = slice(0, hq // hk), slice(0, 1)
    kc = torch.cat([prev[0][:, :, gk], k[:, :, gk]], 1)
    vc = torch.cat([prev[1][:, :, gk], v[:, :, gk]], 1)
    ro, _, rq, rk, rv = O.attention_fwd_bwd(
        lambda q, k, v: O.window_attention(q, k, v, None, (w, 0), True), q[:, :, gq], kc, vc,
        do[:, :, gq])
    _check("c3 own chunk", out[:, :, gq], (qg.grad[:, :, gq], kg.grad[:, :, gk], vg.grad[:, :, gk]),
           ro, (rq, rk[:, s:], rv[:, s:]))
    errs = [_rel(pg.grad[0][:, :, gk], rk[:, :s]), _rel(pg.grad[1][:, :, gk], rv[:, :s])]
    assert max(errs) <= GRAD_TOL, f"c3 previous chunk dk/dv rel-norm {errs}"
    # keys of the previous chunk that no query of this rank can see get exactly zero
    assert pg.grad[:, :, : s - w].abs().max().item() == 0.0
    for t in (out, qg.grad, kg.grad, vg.grad, pg.grad):
        assert torch.isfinite(t.float()).all()


def test_config3_rank_share_on_the_ds_handoff_route(monkeypatch):
    """The same step with the backward's dS hand-off switched on (RSWA_DS_HANDOFF=1: the dK/dV
    kernel stores its 16-bit dS tiles, 2.4 GB here, and the dQ kernel multiplies them with K
    instead of recomputing S and dP; the interface is that of ring_swa/ops/wrap_flash.py:276-327):
    against the oracle, and against the recomputing route -- dK / dV the same bits, dQ to the
    rounding of another summation order."""
    import ring_swa
    from ring_swa.ops.band_attn import bwd_handoff_active

    s, hq, hk, w, cp, rank = 8192, 32, 8, 4096, 8, 1
    q, do = _randn((1, s, hq, D), 0), _randn((1, s, hq, D), 1)
    k, v = _randn((1, s, hk, D), 2), _randn((1, s, hk, D), 3)
    prev = _randn((2, 1, s, hk, D), 4)

    def step():
        qg, kg, vg, pg = (t.clone().requires_grad_() for t in (q, k, v, prev))
        out = ring_swa.ring_rank_share_attn(qg, kg, vg, [pg], w, cp, rank)
        out.backward(do)
        return out.detach(), qg.grad, kg.grad, vg.grad, pg.grad

    plain = step()
    monkeypatch.setenv("RSWA_DS_HANDOFF", "1")
    assert bwd_handoff_active(q, prev[0][:, s - w:], second_rows=s, window_size=(w, 0), causal=True)
    out, dq, dk, dv, dprev = step()
    monkeypatch.delenv("RSWA_DS_HANDOFF")
    assert torch.equal(out, plain[0])
    assert torch.equal(dk, plain[2]) and torch.equal(dv, plain[3]) and torch.equal(dprev, plain[4])
    assert _rel(dq, plain[1]) <= 2e-3
    gq, gk = slice(0, hq // hk), slice(0, 1)
    kc = torch.cat([prev[0][:, :, gk], k[:, :, gk]], 1)
    vc = torch.cat([prev[1][:, :, gk], v[:, :, gk]], 1)
    ro, _, rq, rk, rv = O.attention_fwd_bwd(
        lambda q, k, v: O.window_attention(q, k, v, None, (w, 0), True), q[:, :, gq], kc, vc,
        do[:, :, gq])
    _check("c3 hand-off", out[:, :, gq], (dq[:, :, gq], dk[:, :, gk], dv[:, :, gk]),
           ro, (rq, rk[:, s:], rv[:, s:]))
    assert torch.isfinite(dq.float()).all()


def _log_uniform_lengths(total, lo, hi, seed):
    g = torch.Generator().manual_seed(seed)
    lens = []
    while sum(lens) < total:
        x = math.exp(math.log(lo) + torch.rand(1, generator=g).item() * (math.log(hi) - math.log(lo)))
        lens.append(int(x))
    lens[-1] -= sum(lens) - total
    if lens[-1] == 0:
        lens.pop()
    return lens


def test_config4_varlen_rank_slices_total32768_window2048():
    import ring_swa
    from ring_swa.rank_share import ring_comm_times

    total, cp, hq, hk, w = 32768, 4, 32, 8, 2048
    s_loc = total // cp
    lens = _log_uniform_lengths(total, 64, 16384, seed=0)
    cu = [0] + list(itertools.accumulate(lens))
    assert cu[-1] == total
    # sequence boundaries must fall inside chunks and some sequence must cross a chunk edge
    assert any(c % s_loc for c in cu[1:-1])
    assert any(a // s_loc != (b - 1) // s_loc for a, b in zip(cu[:-1], cu[1:]))
    q, do = _randn((total, hq, D), 0), _randn((total, hq, D), 1)
    k, v = _randn((total, hk, D), 2), _randn((total, hk, D), 3)
    hops = ring_comm_times(w, s_loc, cp)
    outs, dqs = [], []
    dk, dv = torch.zeros(total, hk, D, device="cuda"), torch.zeros(total, hk, D, device="cuda")
    for r in range(cp):
        sl = slice(r * s_loc, (r + 1) * s_loc)
        qr, kr, vr = (t[sl].clone().requires_grad_() for t in (q, k, v))
        prev = []
        for i in range(1, hops + 1):
            if r - i >= 0:
                ps = slice((r - i) * s_loc, (r - i + 1) * s_loc)
                prev.append(torch.stack([k[ps], v[ps]]).requires_grad_())
        out = ring_swa.ring_rank_share_attn_varlen(qr, kr, vr, prev, w, cu, cp, r)
        out.backward(do[sl])
        outs.append(out.detach())
        dqs.append(qr.grad)
        dk[sl] += kr.grad.float()
        dv[sl] += vr.grad.float()
        for i, p in enumerate(prev, start=1):
            ps = slice((r - i) * s_loc, (r - i + 1) * s_loc)
            dk[ps] += p.grad[0].float()
            dv[ps] += p.grad[1].float()
    out, dq = torch.cat(outs, 0), torch.cat(dqs, 0)
    gq, gk = slice(0, hq // hk), slice(0, 1)
    ro, _, rq, rk, rv = O.attention_fwd_bwd(
        lambda q, k, v: O.sliding_window_attn_varlen(q, k, v, w, cu), q[:, gq], k[:, gk], v[:, gk],
        do[:, gq])
    _check("c4", out[:, gq], (dq[:, gq], dk[:, gk], dv[:, gk]), ro, (rq, rk, rv))
    # and the reference's own invariant: the slices put together equal the single call
    glob = ring_swa.ring_sliding_window_attn_varlen(
        q, k, v, w, torch.tensor(cu, dtype=torch.int32, device="cuda"), cp_size=1)
    assert (out.float() - glob.float()).abs().max().item() <= OUT_TOL
    for t in (out, dq, dk, dv):
        assert torch.isfinite(t.float()).all()


@pytest.mark.parametrize("impl,n_sink,off", [("split", 4, 0), ("fused", 4, 0), ("split", 1, 0),
                                             ("fused", 4, 37), ("split", 4, 37), ("fused", 1, 37)])
def test_config5_streaming_llm_varlen_total65536_sinks(impl, n_sink, off):
    """n_sink = 4: the configuration as stated (keyword-only extension of the API);
    n_sink = 1: the reference's own single sink through the unchanged signature.
    off = 0: sequence boundaries on multiples of 1024, hence on the kernels' tile edges;
    off = 37: boundaries at 1024 c + 37, + 101, + 165 -- inside 32-, 64-, 128- and 256-row tiles."""
    import ring_swa

    total, hq, hk, w = 65536, 32, 8, 4092
    g = torch.Generator().manual_seed(0)
    cuts = sorted((torch.randperm(total // 1024 - 1, generator=g)[:3] + 1).tolist())
    cu = [0] + [c * 1024 + (off + 64 * i if off else 0) for i, c in enumerate(cuts)] + [total]
    assert all((c % 32 != 0) for c in cu[1:-1]) or off == 0
    q, do = _randn((total, hq, D), 0), _randn((total, hq, D), 1)
    k, v = _randn((total, hk, D), 2), _randn((total, hk, D), 3)
    for c in cu[:-1]:
        # every sequence starts with the same sink rows (the reference's precondition,
        # test/test_ring_slm_varlen.py:145-147), keys scaled for peaked softmax mass
        for t in (q, k, v):
            t[c:c + n_sink] = t[:n_sink]
    for c in cu[:-1]:
        k[c:c + n_sink] *= 4
    cu_dev = torch.tensor(cu, dtype=torch.int32, device="cuda")
    qg, kg, vg = (t.clone().requires_grad_() for t in (q, k, v))
    kw = {} if n_sink == 1 else {"num_sink_tokens": n_sink}
    out = ring_swa.ring_streaming_llm_attn_varlen(qg, kg, vg, w, cu_dev, cp_size=1, impl=impl, **kw)
    out.backward(do)
    gq, gk = slice(0, hq // hk), slice(0, 1)
    # the oracle one sequence at a time (score matrices of the longest sequence: GBs)
    for a, b in zip(cu[:-1], cu[1:]):
        ro, _, rq, rk, rv = O.attention_fwd_bwd(
            lambda q, k, v: O.streaming_llm_attn(q, k, v, w, n_sink=n_sink),
            q[None, a:b, gq], k[None, a:b, gk], v[None, a:b, gk], do[None, a:b, gq])
        _check(f"c5 {impl} seq [{a},{b})", out[None, a:b, gq],
               (qg.grad[None, a:b, gq], kg.grad[None, a:b, gk], vg.grad[None, a:b, gk]),
               ro, (rq, rk, rv))
        del ro, rq, rk, rv
        torch.cuda.empty_cache()
    for t in (out, qg.grad, kg.grad, vg.grad):
        assert torch.isfinite(t.float()).all()
