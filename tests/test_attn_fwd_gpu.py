"""GPU parity of the HIP forward attention kernel (through the C ABI) against
the CPU oracle.  Tolerances are the ones stated for this path: out max-abs
<= 2e-2 (bf16), LSE <= 1e-3 against an fp32 evaluation of the same mask."""
import itertools

import pytest
import torch

from oracle import attention_oracle as O

pytestmark = pytest.mark.gpu

OUT_TOL = 2e-2
LSE_TOL = 1e-3


def _rand(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g).to(dtype)


def _check(out, lse, ref_o, ref_l):
    out = out.float().cpu()
    lse = lse.float().cpu()
    assert not torch.isnan(out).any()
    err_o = (out - ref_o).abs().max().item()
    fin = torch.isfinite(ref_l)
    assert torch.equal(torch.isfinite(lse), fin), "empty-row pattern differs"
    assert torch.all(lse[~fin] == float("-inf"))
    err_l = (lse[fin] - ref_l[fin]).abs().max().item() if fin.any() else 0.0
    assert err_o <= OUT_TOL, f"out max-abs {err_o}"
    assert err_l <= LSE_TOL, f"lse max-abs {err_l}"


DENSE_CASES = [
    # (B, Sq, Sk, Hq, Hkv, D, window, causal, n_sink)
    (1, 100, 100, 8, 2, 64, (50, 50), False, 0),     # test/test_local_swa.py:98-105
    (1, 1024, 1024, 8, 2, 64, (128, 0), True, 1),    # test/test_local_slm.py:76-84
    (2, 300, 300, 4, 4, 128, (37, 0), True, 0),
    (1, 257, 257, 4, 1, 128, (-1, -1), False, 0),
    (1, 130, 130, 2, 2, 128, (0, 0), True, 0),       # w = 0: own key only
    (1, 200, 333, 4, 2, 128, (40, 0), True, 0),      # Sq < Sk, bottom-right aligned
    (1, 333, 200, 4, 2, 128, (40, 0), True, 0),      # Sq > Sk: leading rows empty
    (1, 333, 200, 2, 2, 128, (-1, -1), False, 0),
    (1, 96, 160, 2, 1, 128, (0, 4096), False, 0),    # ring upper-right triangle block
    (1, 160, 160, 2, 1, 128, (70, 160), False, 0),   # ring skip-lower-left block
    (1, 190, 64, 2, 1, 128, (10, 4096), False, 0),   # Sq > Sk with left window
    (2, 700, 700, 4, 2, 128, (100, 0), True, 4),     # 4 sinks
    (1, 700, 700, 2, 2, 64, (100, 0), True, 1),
    (1, 513, 513, 2, 2, 128, (1000, 0), True, 2),    # window wider than the sequence
    (1, 2048, 2048, 4, 2, 128, (500, 0), True, 0),
    (1, 1, 1, 1, 1, 128, (5, 0), True, 0),
]


@pytest.mark.parametrize("case", DENSE_CASES, ids=lambda c: "x".join(str(x) for x in c))
def test_fwd_dense_matches_oracle(case):
    from ring_swa.ops import wrapped_flash_attn_fwd

    b, sq, sk, hq, hk, d, window, causal, ns = case
    q = _rand((b, sq, hq, d), torch.bfloat16, 1)
    k = _rand((b, sk, hk, d), torch.bfloat16, 2)
    v = _rand((b, sk, hk, d), torch.bfloat16, 3)
    scale = d ** -0.5
    ref_o, ref_l = O.window_attention(q, k, v, scale, window, causal, ns)
    out, lse = wrapped_flash_attn_fwd(q.cuda(), k.cuda(), v.cuda(), scale, window, causal,
                                      num_sink=ns)
    torch.cuda.synchronize()
    assert out.shape == q.shape and out.dtype == q.dtype
    assert lse.shape == (b, hq, sq) and lse.dtype == torch.float32
    _check(out, lse, ref_o, ref_l)


def test_fwd_fp16_and_custom_scale():
    from ring_swa.ops import wrapped_flash_attn_fwd

    q = _rand((1, 150, 4, 128), torch.float16, 1)
    k = _rand((1, 150, 2, 128), torch.float16, 2)
    v = _rand((1, 150, 2, 128), torch.float16, 3)
    ref_o, ref_l = O.window_attention(q, k, v, 0.2, (33, 0), True)
    out, lse = wrapped_flash_attn_fwd(q.cuda(), k.cuda(), v.cuda(), 0.2, (33, 0), True)
    _check(out, lse, ref_o, ref_l)


def test_fwd_strided_views():
    """Slices the callers pass: q[:, 1:], k[:, 1:] (ring_swa/streaming_llm/naive.py:21-28)
    and q[:, :v], kv[:, :, -v:] (ring_swa/sliding_window/nonvarlen.py:139-142)."""
    from ring_swa.ops import wrapped_flash_attn_fwd

    q = _rand((2, 201, 4, 128), torch.bfloat16, 1)
    kv = _rand((2, 2, 201, 2, 128), torch.bfloat16, 2)
    dq, dkv = q.cuda(), kv.cuda()
    ref_o, ref_l = O.window_attention(q[:, 1:], kv[0][:, 1:], kv[1][:, 1:], None, (20, 0), True)
    out, lse = wrapped_flash_attn_fwd(dq[:, 1:], dkv[0][:, 1:], dkv[1][:, 1:], None, (20, 0), True)
    _check(out, lse, ref_o, ref_l)
    vl = 77
    ref_o, ref_l = O.window_attention(q[:, :vl], kv[0][:, -vl:], kv[1][:, -vl:], None, (0, 201),
                                      False)
    out, lse = wrapped_flash_attn_fwd(dq[:, :vl], dkv[0][:, -vl:], dkv[1][:, -vl:], None, (0, 201),
                                      False)
    _check(out, lse, ref_o, ref_l)


@pytest.mark.parametrize("lens,window,ns", [
    ([5, 130, 64, 1, 300], (50, 0), 0),
    ([257, 255], (-1, 0), 0),
    ([100, 400, 129], (64, 0), 1),
    ([100, 400, 129], (64, 0), 4),
])
def test_fwd_varlen_matches_oracle(lens, window, ns):
    from ring_swa.ops import wrapped_flash_attn_fwd_varlen

    cu = torch.tensor([0] + list(itertools.accumulate(lens)), dtype=torch.int32)
    t = int(cu[-1])
    q = _rand((t, 4, 128), torch.bfloat16, 1)
    k = _rand((t, 2, 128), torch.bfloat16, 2)
    v = _rand((t, 2, 128), torch.bfloat16, 3)
    ref_o, ref_l = O.window_attention_varlen(q, k, v, cu, cu, None, window, True, ns)
    out, lse = wrapped_flash_attn_fwd_varlen(q.cuda(), k.cuda(), v.cuda(), None, window,
                                             cu.cuda(), cu.cuda(), max(lens), max(lens), True,
                                             num_sink=ns)
    assert out.shape == q.shape and lse.shape == (4, t)
    _check(out, lse, ref_o, ref_l)


def test_fwd_varlen_different_q_and_k_segmentation():
    """Packed call with q and k cut differently (the per-sequence sink backward of
    ring_swa/streaming_llm/naive.py:181-206 uses one key per sequence)."""
    from ring_swa.ops import wrapped_flash_attn_fwd_varlen

    lens_q, lens_k = [70, 200, 3], [1, 1, 1]
    cu_q = torch.tensor([0] + list(itertools.accumulate(lens_q)), dtype=torch.int32)
    cu_k = torch.tensor([0] + list(itertools.accumulate(lens_k)), dtype=torch.int32)
    q = _rand((int(cu_q[-1]), 4, 128), torch.bfloat16, 1)
    k = _rand((3, 2, 128), torch.bfloat16, 2)
    v = _rand((3, 2, 128), torch.bfloat16, 3)
    ref_o, ref_l = O.window_attention_varlen(q, k, v, cu_q, cu_k, None, (-1, -1), False)
    out, lse = wrapped_flash_attn_fwd_varlen(q.cuda(), k.cuda(), v.cuda(), None, (-1, -1),
                                             cu_q.cuda(), cu_k.cuda(), 200, 1, False)
    _check(out, lse, ref_o, ref_l)


def test_fwd_split_kv_merge_invariance():
    """attention(A u B) == merge(attention(A), attention(B)) on the GPU kernels:
    ties the kernel's LSE to the merge kernel without any oracle."""
    from ring_swa.ops import merge_attn_out, wrapped_flash_attn_fwd

    q = _rand((1, 256, 4, 128), torch.bfloat16, 1).cuda()
    k = _rand((1, 512, 2, 128), torch.bfloat16, 2).cuda()
    v = _rand((1, 512, 2, 128), torch.bfloat16, 3).cuda()
    full_o, full_l = wrapped_flash_attn_fwd(q, k, v, None, (-1, -1), False)
    oa, la = wrapped_flash_attn_fwd(q, k[:, :200], v[:, :200], None, (-1, -1), False)
    ob, lb = wrapped_flash_attn_fwd(q, k[:, 200:], v[:, 200:], None, (-1, -1), False)
    acc = oa.float()
    merge_attn_out(acc, la, ob, lb)
    assert (acc - full_o.float()).abs().max().item() <= OUT_TOL
    assert (la - full_l).abs().max().item() <= LSE_TOL


def test_fwd_rejects_bad_arguments():
    from ring_swa.ops import wrapped_flash_attn_fwd

    q = torch.zeros(1, 8, 4, 128, dtype=torch.bfloat16, device="cuda")
    k = torch.zeros(1, 8, 3, 128, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(AssertionError):
        wrapped_flash_attn_fwd(q, k, k, None, (1, 0), True)          # 4 % 3 != 0
    q96 = torch.zeros(1, 8, 4, 96, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(NotImplementedError):
        wrapped_flash_attn_fwd(q96, q96, q96, None, (1, 0), True)     # head_dim 96
    qf = torch.zeros(1, 8, 4, 128, device="cuda")
    with pytest.raises(NotImplementedError):
        wrapped_flash_attn_fwd(qf, qf, qf, None, (1, 0), True)        # fp32
    with pytest.raises(ValueError):
        wrapped_flash_attn_fwd(q, q, q, -1.0, (1, 0), True)           # scale <= 0


def test_fwd_without_any_key_gives_the_empty_row_pair():
    """An empty KV slice: every row is empty, out = 0 and lse = -inf (the merge identity),
    the same convention the backward assumes for it."""
    from ring_swa.ops import attn_bwd, attn_fwd

    q = torch.randn(2, 37, 4, 128, device="cuda").bfloat16()
    k = torch.empty(2, 0, 2, 128, device="cuda", dtype=torch.bfloat16)
    out, lse = attn_fwd(q, k, k.clone(), None, (16, 0), True)
    assert out.shape == q.shape and (out == 0).all()
    assert lse.shape == (2, 4, 37) and torch.isinf(lse).all() and (lse < 0).all()
    dq, dk, dv = torch.full_like(q, 3.0), torch.empty_like(k), torch.empty_like(k)
    attn_bwd(q, k, k.clone(), out, lse, torch.ones_like(q), dq, dk, dv, None, (16, 0), True)
    torch.cuda.synchronize()
    assert (dq == 0).all()


@pytest.mark.parametrize("case", [
    # (B, Sq, Sk, Hq, Hkv, D, window, causal, dtype): a second block merged into the result of a first
    (1, 512, 512, 4, 2, 128, (0, 512), False, torch.bfloat16),    # previous-chunk corner
    (2, 300, 200, 4, 4, 64, (-1, -1), False, torch.bfloat16),
    (1, 777, 500, 2, 1, 128, (100, 50), False, torch.float16),    # rows with no key in the block
    (1, 200, 333, 6, 2, 64, (40, 0), True, torch.bfloat16),
], ids=["corner", "full", "two_sided_f16", "causal_sq_lt_sk"])
def test_fwd_accumulate_into_equals_forward_plus_merge(case):
    """out_accumulate of the ABI: the block merged into running (out, lse) in the forward's
    epilogue must give the bits of a forward into temporaries followed by the merge kernel;
    rows that the running result, the block, or both leave empty included."""
    from ring_swa.ops import attn_fwd, merge_attn_out

    b, sq, sk, hq, hk, d, window, causal, dtype = case
    torch.manual_seed(9)
    q = torch.randn(b, sq, hq, d, device="cuda").to(dtype)
    k1, v1 = (torch.randn(b, sq, hk, d, device="cuda").to(dtype) for _ in range(2))
    k2, v2 = (torch.randn(b, sk, hk, d, device="cuda").to(dtype) for _ in range(2))
    # running result: a causal band of width 64 over the first keys -- with sq > 64 ... some
    # rows are empty only if the mask says so; make the first 5 rows empty on purpose
    out0, lse0 = attn_fwd(q, k1, v1, None, (64, 0), True)
    out0[:, :5] = 0
    lse0[:, :, :5] = float("-inf")
    ref_out, ref_lse = out0.clone(), lse0.clone()
    o2, l2 = attn_fwd(q, k2, v2, None, window, causal)
    merge_attn_out(ref_out, ref_lse, o2, l2)
    got_out, got_lse = out0.clone(), lse0.clone()
    r = attn_fwd(q, k2, v2, None, window, causal, accumulate_into=(got_out, got_lse))
    assert r[0] is got_out and r[1] is got_lse
    assert torch.equal(got_lse, ref_lse)
    assert torch.equal(got_out, ref_out)
    # views: only a row range of a larger running result
    big_out, big_lse = out0.clone(), lse0.clone()
    n = sq // 2
    attn_fwd(q[:, :n], k2, v2, None, window, causal, mask_shift=sk - sq,
             accumulate_into=(big_out[:, :n], big_lse[:, :, :n]))
    assert torch.equal(big_out[:, n:], out0[:, n:]) and torch.equal(big_lse[:, :, n:], lse0[:, :, n:])
    assert torch.equal(big_out[:, :n], ref_out[:, :n]) and torch.equal(big_lse[:, :, :n], ref_lse[:, :, :n])
