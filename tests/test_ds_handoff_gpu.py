"""GPU parity of the backward's dS hand-off route (``ds_handoff`` of the C ABI): the dK/dV
kernel stores its 16-bit dS tiles, dQ comes from a kernel that multiplies them with K.  Checked
against the CPU oracle on the same seeded inputs (gradients within 1e-2 relative norm plus the
elementwise bound of tests/gradcheck_util.py; the path's stated tolerance is 5e-2), and against
the recomputing route: dK / dV bit for bit (the same kernel body writes them), dQ within the
16-bit rounding of two different summation orders."""
import pytest
import torch

from oracle import attention_oracle as O

pytestmark = pytest.mark.gpu

from gradcheck_util import GRAD_TOL, relnorm  # noqa: E402


def _rand(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g).to(dtype)


def _bwd(q, k, v, o, lse, do, scale, window, causal, handoff, cu=None, second=None, ns=0,
         poison=True, dq_init=None):
    """One backward through the C ABI into fresh (NaN-filled) buffers."""
    from ring_swa.ops.band_attn import attn_bwd, bwd_handoff_active

    fill = float("nan") if poison else 0.0
    gq = torch.full_like(q, fill) if dq_init is None else dq_init.clone()
    gk, gv = torch.full_like(k, fill), torch.full_like(v, fill)
    sec = None
    if second is not None:
        g2k, g2v = torch.full_like(second[0], fill), torch.full_like(second[1], fill)
        sec = (second[0], second[1], g2k, g2v)
    attn_bwd(q, k, v, o, lse, do, gq, gk, gv, scale, window, causal, cu, cu, num_sink=ns,
             second=sec, handoff=handoff, dq_accumulate=dq_init is not None)
    torch.cuda.synchronize()
    rows2 = 0 if second is None else second[0].shape[1]
    active = bwd_handoff_active(q, k, cu, cu, second_rows=rows2, window_size=window, causal=causal,
                                num_sink=ns, handoff=handoff)
    return (gq, gk, gv) + ((sec[2], sec[3]) if sec else ()), active


DENSE = [
    # (B, Sq, Sk, Hq, Hkv, D, window, causal)
    (1, 1024, 1024, 8, 2, 128, (300, 0), True),      # 4 q heads per kv head: 4 heads per block
    (2, 700, 700, 4, 2, 128, (100, 0), True),        # 2 heads per block, ragged tiles
    (1, 900, 900, 3, 3, 128, (257, 0), True),        # 1 head per block (256-row blocks)
    (1, 1500, 1500, 6, 2, 64, (512, 0), True),       # odd group, head_dim 64
    (1, 2048, 2048, 8, 1, 128, (1000, 0), True),     # group 8: two 4-head blocks per tile
    (1, 513, 513, 4, 4, 128, (-1, -1), True),        # plain causal: every key block of the sequence
    (1, 300, 300, 4, 1, 128, (-1, -1), False),       # no mask at all
    (1, 640, 640, 4, 2, 128, (70, 40), False),       # two-sided window
    (1, 333, 777, 4, 2, 128, (200, 0), True),        # more keys than queries (bottom-right aligned)
    (1, 777, 333, 4, 2, 128, (200, 0), True),        # leading rows see nothing
    (1, 96, 4096, 4, 1, 128, (3000, 0), True),       # few rows, long window
    (1, 1, 1, 1, 1, 128, (5, 0), True),
    (1, 31, 33, 2, 1, 64, (0, 0), True),             # one key per row
    (1, 2100, 2100, 4, 1, 128, (31, 0), True),       # window shorter than a row tile
    (3, 257, 257, 2, 2, 128, (255, 1), False),
]


@pytest.mark.parametrize("case", DENSE, ids=lambda c: "x".join(str(x) for x in c))
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
def test_handoff_dense_matches_oracle_and_recompute(case, dtype):
    from ring_swa.ops import attn_fwd

    b, sq, sk, hq, hk, d, window, causal = case
    if dtype == torch.float16 and case not in DENSE[:4]:
        pytest.skip("fp16 on the first cases only")
    q, do = _rand((b, sq, hq, d), dtype, 1), _rand((b, sq, hq, d), dtype, 4)
    k, v = _rand((b, sk, hk, d), dtype, 2), _rand((b, sk, hk, d), dtype, 3)
    scale = d ** -0.5
    _, _, rq, rk, rv = O.attention_fwd_bwd(
        lambda q, k, v: O.window_attention(q, k, v, scale, window, causal, 0), q, k, v, do)
    qc, kc, vc, dc = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    out, lse = attn_fwd(qc, kc, vc, scale, window, causal)
    # ("force": these launches are small enough for the dK/dV kernel to split their key tiles
    # over several blocks, which keeps the recomputing route unless the hand-off is preferred)
    (hq_, hk_, hv_), active = _bwd(qc, kc, vc, out, lse, dc, scale, window, causal, "force")
    assert active, "the route was expected to be taken"
    (bq, bk, bv), _ = _bwd(qc, kc, vc, out, lse, dc, scale, window, causal, False)
    errs = [relnorm(g, r) for g, r in ((hq_, rq), (hk_, rk), (hv_, rv))]
    assert max(errs) <= GRAD_TOL, f"rel-norm errors dq/dk/dv = {errs}"
    # dK / dV: the same sums in the same order wherever the recomputing route did not split
    if (sk + 255) // 256 * hk * b >= 129 or hq == hk:
        assert torch.equal(hk_, bk) and torch.equal(hv_, bv), "dK / dV differ between the routes"
    assert relnorm(hq_, bq.float().cpu()) <= 6e-3, "dQ of the two routes"


def test_route_is_taken_where_expected():
    from ring_swa.ops.band_attn import bwd_handoff_active, bwd_workspace_bytes

    q = torch.empty(1, 8192, 32, 128, dtype=torch.bfloat16, device="cuda")
    k = torch.empty(1, 4096, 8, 128, dtype=torch.bfloat16, device="cuda")
    kw = dict(second_rows=8192, window_size=(4096, 0), causal=True)
    assert bwd_handoff_active(q, k, **kw, handoff=True)
    assert not bwd_handoff_active(q, k, **kw, handoff=None), "not the default (no faster)"
    assert not bwd_handoff_active(q, k, **kw, handoff=False)
    assert not bwd_handoff_active(q, k, **kw, num_sink=4, handoff=True)
    base = bwd_workspace_bytes(q, k, **kw)
    extra = bwd_workspace_bytes(q, k, **kw, handoff=True) - base
    # 32 heads x 256 row tiles x 18 key blocks x 16 KiB
    assert 32 * 256 * 18 * 16384 <= extra <= 32 * 256 * 18 * 16384 + 4096


PACKED = [
    # (lengths, Hq, Hkv, D, window)
    ([300, 1, 700, 33, 256, 64], 8, 2, 128, 128),
    ([1000, 24], 4, 4, 128, 300),
    ([5, 6, 7, 1500, 2], 4, 1, 64, 1000),
    ([2048, 2048], 8, 2, 128, 2000),
    ([100] * 30, 4, 2, 128, 64),
]


@pytest.mark.parametrize("case", PACKED, ids=lambda c: f"{len(c[0])}seq-{c[1]}x{c[2]}x{c[3]}-w{c[4]}")
def test_handoff_packed_matches_oracle(case):
    from ring_swa.ops import attn_fwd

    lens, hq, hk, d, w = case
    t = sum(lens)
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    pad = 5  # rows past the last sequence belong to nobody
    q, do = _rand((t + pad, hq, d), torch.bfloat16, 1), _rand((t + pad, hq, d), torch.bfloat16, 4)
    k, v = _rand((t + pad, hk, d), torch.bfloat16, 2), _rand((t + pad, hk, d), torch.bfloat16, 3)
    scale = d ** -0.5
    _, _, rq, rk, rv = O.attention_fwd_bwd(
        lambda q, k, v: O.window_attention_varlen(q, k, v, cu, cu, scale, (w, 0), True),
        q[:t], k[:t], v[:t], do[:t])
    cu_dev = torch.tensor(cu, dtype=torch.int32, device="cuda")
    qc, kc, vc, dc = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    out, lse = attn_fwd(qc, kc, vc, scale, (w, 0), True, cu_dev, cu_dev)
    (gq, gk, gv), active = _bwd(qc, kc, vc, out, lse, dc, scale, (w, 0), True, "force", cu=cu_dev,
                                poison=False)
    assert active
    errs = [relnorm(g[:t], r) for g, r in ((gq, rq), (gk, rk), (gv, rv))]
    assert max(errs) <= GRAD_TOL, f"rel-norm errors dq/dk/dv = {errs}"


@pytest.mark.parametrize("s,w,hq,hk", [(1024, 512, 8, 2), (768, 300, 4, 4), (2048, 2048 - 256, 4, 1)])
def test_handoff_with_keys_in_two_ranges(s, w, hq, hk):
    """The rank step's band: keys = tail of the previous chunk, then the own chunk."""
    from ring_swa.ops import attn_fwd

    d = 128
    tail = -(-w // 256) * 256
    q, do = _rand((1, s, hq, d), torch.bfloat16, 1), _rand((1, s, hq, d), torch.bfloat16, 4)
    k, v = _rand((1, 2 * s, hk, d), torch.bfloat16, 2), _rand((1, 2 * s, hk, d), torch.bfloat16, 3)
    scale = d ** -0.5
    _, _, rq, rk, rv = O.attention_fwd_bwd(
        lambda q, k, v: O.window_attention(q, k, v, scale, (w, 0), True, 0), q, k, v, do)
    qc, kc, vc, dc = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    k1, v1 = kc[:, s - tail:s], vc[:, s - tail:s]
    k2, v2 = kc[:, s:], vc[:, s:]
    out, lse = attn_fwd(qc, k1, v1, scale, (w, 0), True, second=(k2, v2))
    (gq, gk1, gv1, gk2, gv2), active = _bwd(qc, k1, v1, out, lse, dc, scale, (w, 0), True, "force",
                                            second=(k2, v2))
    assert active
    assert relnorm(gq, rq) <= GRAD_TOL
    assert relnorm(torch.cat([gk1, gk2], 1), rk[:, s - tail:]) <= GRAD_TOL
    assert relnorm(torch.cat([gv1, gv2], 1), rv[:, s - tail:]) <= GRAD_TOL


def test_handoff_dq_accumulate_and_stale_workspace():
    """dq_accumulate adds to what dq holds; a workspace full of NaN changes nothing."""
    from ring_swa.ops import attn_fwd
    from ring_swa.ops.band_attn import attn_bwd, bwd_workspace_bytes

    b, s, hq, hk, d, w = 1, 1536, 8, 2, 128, 400
    q, do = _rand((b, s, hq, d), torch.bfloat16, 1).cuda(), _rand((b, s, hq, d), torch.bfloat16, 4).cuda()
    k, v = _rand((b, s, hk, d), torch.bfloat16, 2).cuda(), _rand((b, s, hk, d), torch.bfloat16, 3).cuda()
    out, lse = attn_fwd(q, k, v, None, (w, 0), True)
    (gq, gk, gv), active = _bwd(q, k, v, out, lse, do, None, (w, 0), True, "force")
    assert active
    init = _rand((b, s, hq, d), torch.bfloat16, 9).cuda()
    (aq, _, _), _ = _bwd(q, k, v, out, lse, do, None, (w, 0), True, "force", dq_init=init)
    assert torch.equal(aq, (init.float() + gq.float()).to(torch.bfloat16))
    need = bwd_workspace_bytes(q, k, window_size=(w, 0), causal=True, handoff="force")
    for fill in (0xFF, 0x7F, 0):
        ws = torch.full((need,), fill, dtype=torch.uint8, device="cuda")
        wq, wk, wv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        attn_bwd(q, k, v, out, lse, do, wq, wk, wv, None, (w, 0), True, workspace=ws, handoff="force")
        assert torch.equal(wq, gq) and torch.equal(wk, gk) and torch.equal(wv, gv)
    # phases one by one on one workspace: statistics, dK/dV (stores dS), dQ (reads it)
    ws = torch.full((need,), 0xFF, dtype=torch.uint8, device="cuda")
    pq, pk, pv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    for ph in (1, 2, 4):
        attn_bwd(q, k, v, out, lse, do, pq, pk, pv, None, (w, 0), True, workspace=ws, phases=ph,
                 handoff="force")
    assert torch.equal(pq, gq) and torch.equal(pk, gk) and torch.equal(pv, gv)


def test_automatic_choice_follows_the_workspace_it_is_given(monkeypatch):
    """With the route switched on by the environment, a call that brings its own workspace takes
    the hand-off only if the dS tiles fit in it; sized without them, the call recomputes (same
    bits as with the route off) instead of failing."""
    from ring_swa.ops import attn_fwd
    from ring_swa.ops.band_attn import attn_bwd, bwd_workspace_bytes

    b, s, hq, hk, d, w = 1, 70000, 8, 8, 128, 300   # 274 key blocks x 8 heads: no split launch
    q, do = _rand((b, s, hq, d), torch.bfloat16, 1).cuda(), _rand((b, s, hq, d), torch.bfloat16, 4).cuda()
    k, v = _rand((b, s, hk, d), torch.bfloat16, 2).cuda(), _rand((b, s, hk, d), torch.bfloat16, 3).cuda()
    out, lse = attn_fwd(q, k, v, None, (w, 0), True)
    ref = [torch.empty_like(t) for t in (q, k, v)]
    attn_bwd(q, k, v, out, lse, do, *ref, None, (w, 0), True, handoff=False)
    monkeypatch.setenv("RSWA_DS_HANDOFF", "1")
    small = bwd_workspace_bytes(q, k, window_size=(w, 0), causal=True, handoff=False)
    large = bwd_workspace_bytes(q, k, window_size=(w, 0), causal=True, handoff=None)
    assert large > small
    got = [torch.empty_like(t) for t in (q, k, v)]
    attn_bwd(q, k, v, out, lse, do, *got, None, (w, 0), True,
             workspace=torch.empty(small, dtype=torch.uint8, device="cuda"))
    assert all(torch.equal(a, b) for a, b in zip(got, ref))
    handed = [torch.empty_like(t) for t in (q, k, v)]
    attn_bwd(q, k, v, out, lse, do, *handed, None, (w, 0), True,
             workspace=torch.empty(large, dtype=torch.uint8, device="cuda"))
    assert torch.equal(handed[1], ref[1]) and torch.equal(handed[2], ref[2])
    assert not torch.equal(handed[0], ref[0])  # another summation order: the route was taken
    assert ((handed[0].float() - ref[0].float()).norm() / ref[0].float().norm()).item() < 2e-3
