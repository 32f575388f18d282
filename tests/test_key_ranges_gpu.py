"""Keys in two row ranges (``seg_rows`` / ``k2 .. dv2`` of the ABI): a block whose keys are
the rows of one tensor followed by the rows of another -- a ring rank's tail of the previous
chunk and its own chunk (ring_swa/sliding_window/nonvarlen.py:95-150 computes them as two
blocks and a merge) -- must give the bits of the same call on the concatenated keys, forward
and backward, and agree with the oracle."""
import pytest
import torch

from oracle import attention_oracle as O

pytestmark = pytest.mark.gpu

from gradcheck_util import GRAD_TOL, relnorm as _relnorm  # noqa: E402

CASES = [
    # (B, Sq, S1, S2, Hq, Hkv, D, window, causal, dtype)
    (1, 512, 256, 512, 4, 2, 128, (256, 0), True, torch.bfloat16),     # tail + own chunk, band
    (2, 300, 512, 300, 4, 4, 64, (200, 0), True, torch.bfloat16),      # ragged second range
    (1, 700, 256, 700, 8, 2, 128, (-1, -1), False, torch.float16),     # full attention
    (1, 1024, 768, 1024, 8, 2, 128, (768, 0), True, torch.bfloat16),   # few key tiles: split dK/dV
    (1, 130, 256, 77, 2, 1, 64, (100, 30), False, torch.bfloat16),     # two-sided window
]


@pytest.mark.parametrize("addressing", ["near", "far"])
@pytest.mark.parametrize("case", CASES, ids=[f"c{i}" for i in range(len(CASES))])
def test_two_key_ranges_equal_concatenated_keys(case, addressing, monkeypatch):
    """(`far`: the kernels that base every tile fetch at the tile's own first row, as the library
    picks them for tensors beyond 2 GiB.)"""
    from ring_swa.ops import attn_bwd, attn_fwd
    from ring_swa.ops.band_attn import bwd_workspace_bytes

    b, sq, s1, s2, hq, hk, d, window, causal, dtype = case
    torch.manual_seed(3)
    q, do = (torch.randn(b, sq, hq, d, device="cuda").to(dtype) for _ in range(2))
    # the two ranges as views with equal strides: rows of two separate [B, S, H, D] buffers
    n = max(s1, s2)
    bufs = [torch.randn(b, n, hk, d, device="cuda").to(dtype) for _ in range(4)]
    k1, v1, k2, v2 = bufs[0][:, :s1], bufs[1][:, :s1], bufs[2][:, :s2], bufs[3][:, :s2]
    kc, vc = torch.cat([k1, k2], 1), torch.cat([v1, v2], 1)

    ref_out, ref_lse = attn_fwd(q, kc, vc, None, window, causal)
    rdq, rdk, rdv = torch.empty_like(q), torch.empty_like(kc), torch.empty_like(vc)
    attn_bwd(q, kc, vc, ref_out, ref_lse, do, rdq, rdk, rdv, None, window, causal)
    if addressing == "far":
        monkeypatch.setenv("RSWA_ADDRESSING", "far")
    out, lse = attn_fwd(q, k1, v1, None, window, causal, second=(k2, v2))
    assert torch.equal(out, ref_out) and torch.equal(lse, ref_lse)

    dq = torch.empty_like(q)
    g = [torch.full_like(t, float("nan")) for t in bufs]
    dk1, dv1, dk2, dv2 = g[0][:, :s1], g[1][:, :s1], g[2][:, :s2], g[3][:, :s2]
    ws = torch.empty(bwd_workspace_bytes(q, k1, second_rows=s2), dtype=torch.uint8, device="cuda")
    attn_bwd(q, k1, v1, out, lse, do, dq, dk1, dv1, None, window, causal, workspace=ws,
             second=(k2, v2, dk2, dv2))
    torch.cuda.synchronize()
    assert torch.equal(dq, rdq)
    assert torch.equal(torch.cat([dk1, dk2], 1), rdk)
    assert torch.equal(torch.cat([dv1, dv2], 1), rdv)
    # nothing outside the two ranges was written
    for t, s in ((g[0], s1), (g[1], s1), (g[2], s2), (g[3], s2)):
        assert torch.isnan(t[:, s:].float()).all()


def test_two_key_ranges_match_the_oracle():
    from ring_swa.ops import attn_bwd, attn_fwd

    torch.manual_seed(4)
    b, s, w, hq, hk, d = 1, 512, 256, 4, 2, 64
    q, do = (torch.randn(b, s, hq, d).bfloat16() for _ in range(2))
    k, v = (torch.randn(b, 2 * s, hk, d).bfloat16() for _ in range(2))
    # rank 1 of 2 under window w: own chunk plus the last w keys of the previous one
    fn = lambda q_, k_, v_: O.sliding_window_attn(q_, k_, v_, w)
    qg = torch.cat([torch.zeros_like(q), q], 1)
    dog = torch.cat([torch.zeros_like(do), do], 1)
    ro, rl, rq, rk, rv = O.attention_fwd_bwd(fn, qg, k, v, dog)
    qd, dod, kd, vd = q.cuda(), do.cuda(), k.cuda(), v.cuda()
    tail = slice(s - w, s)
    out, lse = attn_fwd(qd, kd[:, tail], vd[:, tail], None, (w, 0), True,
                        second=(kd[:, s:], vd[:, s:]))
    assert (out.float().cpu() - ro[:, s:]).abs().max().item() <= 2e-2
    assert (lse.cpu() - rl[:, :, s:]).abs().max().item() <= 1e-3
    dq, dk, dv = torch.empty_like(qd), torch.zeros_like(kd), torch.zeros_like(vd)
    attn_bwd(qd, kd[:, tail], vd[:, tail], out, lse, dod, dq, dk[:, tail], dv[:, tail], None,
             (w, 0), True, second=(kd[:, s:], vd[:, s:], dk[:, s:], dv[:, s:]))
    torch.cuda.synchronize()
    assert _relnorm(dq, rq[:, s:]) <= GRAD_TOL
    # (the zero rows of qg and dog contribute nothing to the oracle's dk / dv)
    assert _relnorm(dk[:, s - w:], rk[:, s - w:]) <= GRAD_TOL
    assert _relnorm(dv[:, s - w:], rv[:, s - w:]) <= GRAD_TOL


@pytest.mark.parametrize("s_loc,w,cp,batch", [(512, 256, 3, 1), (1024, 768, 2, 1), (768, 512, 2, 2),
                                              (512, 300, 3, 2), (1024, 1, 2, 1), (768, 513, 2, 1)])
def test_rank_share_as_one_band_pass(s_loc, w, cp, batch, monkeypatch):
    """A rank whose window is shorter than a chunk (and, rounded up to 256 rows, no longer than
    it) runs [tail of the previous chunk | own chunk] as one band pass over two key ranges (ring_swa/sliding_window/nonvarlen.py:95-150 runs two
    blocks and merges).  The shares of all ranks put together must equal the oracle on the whole
    sequence, gradients of the previous chunk included (zero outside the tail), and the step
    must agree with the two-block form of the same step."""
    import ring_swa
    from ring_swa import rank_share

    hq, hk, d = 4, 2, 128
    total = s_loc * cp
    g = torch.Generator().manual_seed(21)
    q, do = (torch.randn(batch, total, hq, d, generator=g).bfloat16() for _ in range(2))
    k, v = (torch.randn(batch, total, hk, d, generator=g).bfloat16() for _ in range(2))
    ref = O.attention_fwd_bwd(lambda q, k, v: O.sliding_window_attn(q, k, v, w), q, k, v, do)

    taken = []
    plain = rank_share._one_pass

    def share(one_pass):
        monkeypatch.setattr(rank_share, "_one_pass", (lambda *a: taken.append(plain(*a)) or taken[-1])
                            if one_pass else (lambda *a: None))
        outs, dqs = [], []
        dk, dv = torch.zeros(batch, total, hk, d), torch.zeros(batch, total, hk, d)
        for r in range(cp):
            sl = slice(r * s_loc, (r + 1) * s_loc)
            qr, kr, vr = (t[:, sl].cuda().requires_grad_() for t in (q, k, v))
            prev = []
            if r > 0:
                ps = slice((r - 1) * s_loc, r * s_loc)
                prev.append(torch.stack([k[:, ps], v[:, ps]]).cuda().requires_grad_())
            out = ring_swa.ring_rank_share_attn(qr, kr, vr, prev, w, cp, r)
            out.backward(do[:, sl].cuda())
            outs.append(out.detach().float().cpu())
            dqs.append(qr.grad.float().cpu())
            dk[:, sl] += kr.grad.float().cpu()
            dv[:, sl] += vr.grad.float().cpu()
            for p in prev:
                assert not p.grad[:, :, :s_loc - w].any()  # rows no query of this rank sees
                dk[:, ps] += p.grad[0].float().cpu()
                dv[:, ps] += p.grad[1].float().cpu()
        return torch.cat(outs, 1), torch.cat(dqs, 1), dk, dv

    one = share(True)
    # every rank but the first took the one-pass route, forward and backward
    assert len([t for t in taken if t is not None]) == 2 * (cp - 1) and len(taken) == 2 * cp - 1
    two = share(False)
    ro, _, rq, rk, rv = ref
    assert (one[0] - ro).abs().max().item() <= 2e-2
    errs = [_relnorm(a, b) for a, b in zip(one[1:], (rq, rk, rv))]
    assert max(errs) <= GRAD_TOL, f"rel-norm dq/dk/dv = {errs}"
    assert (one[0] - two[0]).abs().max().item() <= 2e-2
    assert max(_relnorm(a, b) for a, b in zip(one[1:], two[1:])) <= GRAD_TOL
