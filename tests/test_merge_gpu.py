"""GPU parity of the HIP LSE-merge kernel (through the C ABI) against the oracle."""
import pytest
import torch

from oracle import attention_oracle as O

pytestmark = pytest.mark.gpu


def _mk(b, s, h, d, o_dt, l_dt, on_dt, ln_dt, seed=0, dev="cuda"):
    g = torch.Generator().manual_seed(seed)
    o = torch.randn(b, s, h, d, generator=g).to(o_dt)
    on = torch.randn(b, s, h, d, generator=g).to(on_dt)
    l = (torch.randn(b, h, s, generator=g) * 3).to(l_dt)
    ln = (torch.randn(b, h, s, generator=g) * 3).to(ln_dt)
    return o, l, on, ln


DT = {
    "ring": (torch.float32, torch.float64, torch.bfloat16, torch.float32),
    "naive": (torch.bfloat16, torch.float32, torch.bfloat16, torch.float32),
    "f32": (torch.float32, torch.float32, torch.float32, torch.float32),
    "f16": (torch.float16, torch.float32, torch.float16, torch.float32),
    "f32_f16": (torch.float32, torch.float64, torch.float16, torch.float64),
}


def _tol(o_dt):
    # one rounding of the stored result: bf16 has 8 bits of mantissa, fp16 11
    return {torch.float32: 2e-6, torch.bfloat16: 2e-2, torch.float16: 4e-3}[o_dt]


@pytest.mark.parametrize("kind", list(DT))
@pytest.mark.parametrize("shape", [(2, 257, 3, 128), (1, 64, 8, 64), (1, 5, 1, 8), (3, 100, 2, 96)])
def test_merge_matches_oracle(kind, shape):
    from ring_swa.ops import merge_attn_out

    o, l, on, ln = _mk(*shape, *DT[kind])
    ref_o, ref_l = O.merge(o.double(), l.double(), on.double(), ln.double())
    do, dl, don, dln = (t.cuda() for t in (o, l, on, ln))
    merge_attn_out(do, dl, don, dln)
    torch.cuda.synchronize()
    assert do.dtype == o.dtype and dl.dtype == l.dtype
    torch.testing.assert_close(do.cpu().double(), ref_o, atol=_tol(o.dtype), rtol=_tol(o.dtype))
    # the reference's own self-test asks 1e-5 on the merged LSE (ring_swa/ops/merge.py:246-250)
    torch.testing.assert_close(dl.cpu().double(), ref_l, atol=1e-5, rtol=0)
    # inputs that are not outputs stay untouched
    assert torch.equal(don.cpu(), on) and torch.equal(dln.cpu(), ln)


def test_merge_at_the_shape_of_the_reference_self_test():
    """ring_swa/ops/merge.py:211-255: batch 8, seq 8192, 16 heads, head_dim 128, running output
    fp32 / LSE fp64, new partial bf16 / fp32, all N(0,1); the reference asks atol = rtol = 1e-2
    on the output and 1e-5 on the LSE.  1 048 576 rows: every block and lane pattern of the
    kernel at full occupancy, which the small cases do not reach.  (The oracle's formula runs
    on the device here: fp64 on 67 million elements.)"""
    from ring_swa.ops import merge_attn_out

    b, s, h, d = 8, 8192, 16, 128
    g = torch.Generator(device="cuda").manual_seed(0)
    o = torch.randn(b, s, h, d, generator=g, device="cuda")
    l = torch.randn(b, h, s, generator=g, device="cuda", dtype=torch.float64)
    on = torch.randn(b, s, h, d, generator=g, device="cuda").bfloat16()
    ln = torch.randn(b, h, s, generator=g, device="cuda")
    ref_o, ref_l = O.merge(o.double(), l, on.double(), ln.double())
    snap_on, snap_ln = on.clone(), ln.clone()
    merge_attn_out(o, l, on, ln)
    torch.cuda.synchronize()
    torch.testing.assert_close(o.double(), ref_o, atol=2e-6, rtol=2e-6)  # (asked: 1e-2)
    torch.testing.assert_close(l, ref_l, atol=1e-5, rtol=1e-5)
    assert torch.equal(on, snap_on) and torch.equal(ln, snap_ln)


def test_merge_identity_and_empty_rows():
    from ring_swa.ops import merge_attn_out

    b, s, h, d = 1, 70, 4, 128
    o, l, on, ln = _mk(b, s, h, d, *DT["ring"])
    # fresh accumulator: zeros / -inf (ring_swa/sliding_window/nonvarlen.py:53-59)
    acc = torch.zeros_like(o).cuda()
    acc_l = torch.full_like(l, float("-inf")).cuda()
    ln[:, :, 3] = float("-inf")  # an empty new row merged into an empty accumulator
    merge_attn_out(acc, acc_l, on.cuda(), ln.cuda())
    want = on.float().clone()
    want[:, 3] = 0
    torch.testing.assert_close(acc.cpu(), want, atol=0, rtol=0)
    assert torch.equal(acc_l.cpu(), ln.double())
    # merging -inf into a filled accumulator changes nothing
    snap_o, snap_l = acc.clone(), acc_l.clone()
    merge_attn_out(acc, acc_l, torch.randn_like(on).cuda(),
                   torch.full_like(ln, float("-inf")).cuda())
    assert torch.equal(acc, snap_o) and torch.equal(acc_l, snap_l)
    assert not torch.isnan(acc).any() and not torch.isnan(acc_l).any()


def test_merge_strided_views():
    """Sliced accumulators as the ring passes them (attn_out[:, :v], lse[:, :, :v]:
    ring_swa/sliding_window/nonvarlen.py:139-148) and the front-padded bf16 pair of
    the naive streaming path (ring_swa/streaming_llm/naive.py:37-39)."""
    from ring_swa.ops import merge_attn_out

    b, s, h, d, v = 2, 96, 4, 128, 40
    o, l, on, ln = _mk(b, s, h, d, *DT["ring"])
    do, dl = o.cuda(), l.cuda()
    don, dln = on[:, :v].contiguous().cuda(), ln[:, :, :v].contiguous().cuda()
    merge_attn_out(do[:, :v], dl[:, :, :v], don, dln)
    ref_o, ref_l = O.merge(o[:, :v].double(), l[:, :, :v].double(), on[:, :v].double(),
                           ln[:, :, :v].double())
    torch.testing.assert_close(do[:, :v].cpu().double(), ref_o, atol=2e-6, rtol=2e-6)
    torch.testing.assert_close(dl[:, :, :v].cpu(), ref_l, atol=1e-5, rtol=0)
    assert torch.equal(do[:, v:].cpu(), o[:, v:]) and torch.equal(dl[:, :, v:].cpu(), l[:, :, v:])
    # expanded (stride-0 batch) new partial
    o2, l2, on2, ln2 = _mk(1, s, h, d, *DT["naive"], seed=3)
    do2, dl2 = o2.cuda().expand(1, s, h, d).clone(), l2.cuda().clone()
    one = on2[:, :1].cuda().expand(1, s, h, d)
    one_l = ln2[:, :, :1].cuda().expand(1, h, s)
    merge_attn_out(do2, dl2, one, one_l)
    ref_o, ref_l = O.merge(o2.double(), l2.double(), on2[:, :1].expand(1, s, h, d).double(),
                           ln2[:, :, :1].expand(1, h, s).double())
    torch.testing.assert_close(do2.cpu().double(), ref_o, atol=2e-2, rtol=2e-2)
    torch.testing.assert_close(dl2.cpu().double(), ref_l, atol=1e-5, rtol=0)


def test_merge_rejects_bad_arguments():
    from ring_swa.ops import merge_attn_out

    o, l, on, ln = (t.cuda() for t in _mk(1, 8, 2, 128, *DT["ring"]))
    with pytest.raises(AssertionError):
        merge_attn_out(o, l.transpose(1, 2), on, ln)
    wide = torch.zeros(1, 8, 2, 256, device="cuda")[..., ::2]  # dim stride 2
    with pytest.raises(NotImplementedError):
        merge_attn_out(wide, l, on, ln)
    with pytest.raises(RuntimeError):
        merge_attn_out(o.cpu(), l.cpu(), on.cpu(), ln.cpu())
