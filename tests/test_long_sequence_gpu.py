"""Sequences whose tensors span more than 2 GiB in one call: 300 000 tokens x 32 q / 8 kv heads
x head_dim 128 (q alone is 2.46 GB; row 262 144 starts at byte 2^31), window 1024, dense and
packed.  The kernels fetch tiles through 32-bit offsets relative to each tile's first row, so
nothing but one tile has to fit them.

The whole problem runs through the public entry points, forward and backward.  A banded
problem is local: the outputs and dQ of rows [a, a + n) depend on keys [a - w, a + n) only, and
dK / dV of keys [a, a + n - w) on those rows only.  One GQA group is checked against the oracle
on such slices -- at the start, across the 2 GiB line, at the end, and (packed) across a
sequence boundary -- to the tolerances of the path: out max-abs 2e-2, LSE 1e-3, gradients
relative norm 1e-2.
"""
import pytest
import torch

from oracle import attention_oracle as O

pytestmark = pytest.mark.gpu

T, HQ, HK, D, W = 300_000, 32, 8, 128, 1024
N = 3072  # rows per checked slice
OUT_TOL, LSE_TOL, GRAD_TOL = 2e-2, 1e-3, 1e-2


def _randn(shape, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.empty(shape, device="cuda", dtype=torch.bfloat16)
    step = 50_000  # generated in pieces: the fp32 draw of a whole tensor would take 5 GB
    for r in range(0, shape[0], step):
        x[r:r + step] = torch.randn((min(step, shape[0] - r),) + tuple(shape[1:]), generator=g,
                                    device="cuda")
    return x


def _rel(x, ref):
    x = x.float()
    assert torch.isfinite(x).all()
    return ((x - ref).norm() / ref.norm().clamp_min(1e-30)).item()


def _check_slice(name, a, seq0, seq1, q, k, v, do, out, lse, dq, dk, dv):
    """Rows [a, a + N) of the sequence [seq0, seq1) (packed row numbers) against the oracle."""
    b = min(a + N, seq1)
    k0 = max(seq0, a - W)
    gq, gk = slice(0, HQ // HK), slice(0, 1)
    ro, rl, rq, rk, rv = O.attention_fwd_bwd(
        lambda q, k, v: O.window_attention(q, k, v, None, (W, 0), True),
        q[None, a:b, gq], k[None, k0:b, gk], v[None, k0:b, gk], do[None, a:b, gq])
    err = (out[a:b, gq].float() - ro[0]).abs().max().item()
    assert err <= OUT_TOL, f"{name}: out max-abs {err}"
    err = (lse[gq, a:b] - rl[0]).abs().max().item()
    assert err <= LSE_TOL, f"{name}: lse max-abs {err}"
    assert _rel(dq[a:b, gq], rq[0]) <= GRAD_TOL, name
    # keys every viewer of which lies inside the slice
    j1 = b if b == seq1 else b - W
    assert j1 - a >= 1024
    errs = [_rel(dk[a:j1, gk], rk[0, a - k0:j1 - k0]), _rel(dv[a:j1, gk], rv[0, a - k0:j1 - k0])]
    assert max(errs) <= GRAD_TOL, f"{name}: dk/dv rel-norm {errs}"


@pytest.mark.parametrize("packed", [False, True], ids=["dense", "packed"])
def test_300k_tokens_window_1024(packed):
    import ring_swa
    from ring_swa.ops import wrapped_flash_attn_fwd, wrapped_flash_attn_fwd_varlen

    q, do = _randn((T, HQ, D), 0), _randn((T, HQ, D), 1)
    k, v = _randn((T, HK, D), 2), _randn((T, HK, D), 3)
    assert q.numel() * 2 > (1 << 31)
    q.requires_grad_(), k.requires_grad_(), v.requires_grad_()
    if packed:
        cu = [0, 140_001, 290_003, T]  # the middle sequence crosses the 2 GiB line
        cu_dev = torch.tensor(cu, dtype=torch.int32, device="cuda")
        out = ring_swa.ring_sliding_window_attn_varlen(q, k, v, W, cu_dev)
        out.backward(do)
        with torch.no_grad():
            _, lse = wrapped_flash_attn_fwd_varlen(q, k, v, D ** -0.5, (W, 0), cu_dev, cu_dev,
                                                   None, None, True)
        o2, dq, dk, dv = out.detach(), q.grad, k.grad, v.grad
        slices = [("first sequence start", 0, 0), ("first sequence end", cu[1] - N, 0),
                  ("second sequence start", cu[1], 1), ("across 2 GiB", (1 << 18) - N // 2, 1),
                  ("last sequence end", T - N, 2)]
    else:
        cu = [0, T]
        out = ring_swa.ring_sliding_window_attn(q[None], k[None], v[None], W)
        out.backward(do[None])
        with torch.no_grad():
            _, lse = wrapped_flash_attn_fwd(q[None], k[None], v[None], D ** -0.5, (W, 0), True)
        o2, lse, dq, dk, dv = out.detach()[0], lse[0], q.grad, k.grad, v.grad
        slices = [("start", 0, 0), ("across 2 GiB", (1 << 18) - N // 2, 0), ("end", T - N, 0)]
    qd, kd, vd = q.detach(), k.detach(), v.detach()
    for name, a, s in slices:
        _check_slice(name, a, cu[s], cu[s + 1], qd, kd, vd, do, o2, lse, dq, dk, dv)
    for t in (o2, dq, dk, dv):
        for r in range(0, T, 100_000):
            assert torch.isfinite(t[r:r + 100_000].float()).all()


@pytest.mark.parametrize("case", [
    dict(sq=777, sk=777, hq=4, hk=2, d=128, window=(100, 0), causal=True, sink=0),
    dict(sq=300, sk=1000, hq=4, hk=4, d=64, window=(-1, -1), causal=True, sink=0),
    dict(sq=1500, sk=1500, hq=8, hk=2, d=128, window=(256, 0), causal=True, sink=4),
    dict(sq=513, sk=640, hq=2, hk=1, d=64, window=(50, 70), causal=False, sink=0),
    dict(packed=[0, 5, 300, 1301, 1302, 2000], hq=4, hk=2, d=128, window=(300, 0), causal=True,
         sink=1),
], ids=["band", "causal_sq_lt_sk", "sinks", "two_sided", "packed_sinks"])
def test_tile_based_addressing_gives_the_same_bits(case, monkeypatch):
    """The kernels that base each tile fetch at the tile's first row (chosen by the library when
    a sequence spans 2 GiB) against the ordinary ones, on the same inputs: same arithmetic, so
    every output bit must agree.  The ordinary ones are checked against the oracle elsewhere."""
    from ring_swa.ops import attn_bwd, attn_fwd

    torch.manual_seed(5)
    d, hq, hk = case["d"], case["hq"], case["hk"]
    mk = lambda *s: torch.randn(*s, device="cuda", dtype=torch.bfloat16)  # noqa: E731
    if "packed" in case:
        cu = torch.tensor(case["packed"], dtype=torch.int32, device="cuda")
        t = case["packed"][-1]
        q, k, v, do = mk(t, hq, d), mk(t, hk, d), mk(t, hk, d), mk(t, hq, d)
    else:
        cu = None
        q, do = mk(2, case["sq"], hq, d), mk(2, case["sq"], hq, d)
        k, v = mk(2, case["sk"], hk, d), mk(2, case["sk"], hk, d)

    def run():
        out, lse = attn_fwd(q, k, v, None, case["window"], case["causal"], cu, cu,
                            num_sink=case["sink"])
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        attn_bwd(q, k, v, out, lse, do, dq, dk, dv, None, case["window"], case["causal"], cu, cu,
                 num_sink=case["sink"])
        return out, lse, dq, dk, dv

    near = run()
    monkeypatch.setenv("RSWA_ADDRESSING", "far")
    far = run()
    for name, x, y in zip(("out", "lse", "dq", "dk", "dv"), near, far):
        assert torch.equal(x, y), name
