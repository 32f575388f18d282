"""The four accumulating block operators (``ring_swa.ops.flash_attn_*_func``, the signatures
and in-place behaviour of ``ring_swa/ops/attn.py:12-196`` upstream) on the HIP kernels against
the oracle: merged into running accumulators of the ring's types (fp32 output, fp64 LSE), into
sliced accumulator views, more query rows than keys (one kernel call when the right window
bound reaches the last key from every row, upstream's two-part route otherwise), packed."""
import pytest
import torch

from gradcheck_util import GRAD_TOL, relnorm
from oracle import attention_oracle as O

pytestmark = pytest.mark.gpu


def _rand(shape, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g).bfloat16()


def _two_part_allowed(sq, sk, window):
    """Upstream's rule for sq > sk: leading rows see every key, the last sk rows the window."""
    allowed = torch.ones(sq, sk, dtype=torch.bool)
    allowed[sq - sk:] = O.window_allowed(sk, sk, window, False)
    return allowed


@pytest.mark.parametrize("sq,sk,window,causal", [
    (200, 200, (37, 0), True),
    (96, 160, (0, 4096), False),
    (190, 64, (10, 4096), False),     # more rows than keys, right bound reaches every key
    (190, 64, (10, 20), False),       # ... and does not: two parts
    (150, 150, (-1, -1), False),
])
def test_dense_forward_merges_into_accumulators_and_backward_fills_buffers(sq, sk, window, causal):
    from ring_swa.ops import flash_attn_bwd_func, flash_attn_fwd_func

    b, hq, hk, d = 2, 4, 2, 128
    q, do = _rand((b, sq, hq, d), 1), _rand((b, sq, hq, d), 4)
    k, v = _rand((b, sk, hk, d), 2), _rand((b, sk, hk, d), 3)
    # a previous partial already sits in the accumulators (keys the block does not contain)
    k0, v0 = _rand((b, 50, hk, d), 5), _rand((b, 50, hk, d), 6)
    two_part = sq > sk and window != (-1, -1) and 0 <= window[1] < sq - 1
    allowed = _two_part_allowed(sq, sk, window) if two_part else O.window_allowed(sq, sk, window, causal)
    full0 = torch.ones(sq, 50, dtype=torch.bool)

    def whole(q, k, v, k0, v0):
        o1, l1 = O.masked_attention(q, k, v, allowed, None)
        o0, l0 = O.masked_attention(q, k0, v0, full0, None)
        return O.merge(o0, l0, o1, l1)

    o_ref, l_ref = whole(q.float(), k.float(), v.float(), k0.float(), v0.float())
    qc, kc, vc, doc = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    o0, l0 = O.masked_attention(q.float(), k0.float(), v0.float(), full0, None)
    # accumulators with spare rows around them: the operator gets views
    acc = torch.full((b, sq + 7, hq, d), 9.0, device="cuda")
    lacc = torch.full((b, hq, sq + 7), 9.0, dtype=torch.float64, device="cuda")
    acc[:, 3:3 + sq], lacc[:, :, 3:3 + sq] = o0.cuda(), l0.double().cuda()
    kv = torch.stack([kc, vc])
    flash_attn_fwd_func(qc, kv, d ** -0.5, window, causal, acc[:, 3:3 + sq], lacc[:, :, 3:3 + sq])
    torch.cuda.synchronize()
    assert (acc[:, :3] == 9).all() and (acc[:, 3 + sq:] == 9).all() and (lacc[:, :, :3] == 9).all()
    assert (acc[:, 3:3 + sq].cpu() - o_ref).abs().max().item() <= 2e-2
    assert (lacc[:, :, 3:3 + sq].float().cpu() - l_ref).abs().max().item() <= 1e-3

    # backward of the block alone, from the block's own statistics
    o_blk, l_blk = O.masked_attention(q.float(), k.float(), v.float(), allowed, None)
    rq, rk, rv = O.attention_bwd_from_stats(q.float(), k.float(), v.float(), o_blk, l_blk,
                                            do.float(), allowed, None)
    dq = torch.full_like(qc, float("nan"))
    dkv = torch.full_like(kv, float("nan"))
    flash_attn_bwd_func(qc, kv, o_blk.bfloat16().cuda(), l_blk.cuda(), doc, dq, dkv, d ** -0.5,
                        window, causal)
    torch.cuda.synchronize()
    errs = [relnorm(dq, rq), relnorm(dkv[0], rk), relnorm(dkv[1], rv)]
    assert max(errs) <= GRAD_TOL, errs


def test_packed_operators():
    from ring_swa.ops import flash_attn_varlen_bwd_func, flash_attn_varlen_fwd_func

    hq, hk, d, w = 4, 2, 128, 30
    cu = [0, 45, 46, 200, 333]
    total = cu[-1]
    q, do = _rand((total, hq, d), 1), _rand((total, hq, d), 4)
    k, v = _rand((total, hk, d), 2), _rand((total, hk, d), 3)
    ro, rl, rq, rk, rv = O.attention_fwd_bwd(
        lambda q, k, v: O.window_attention_varlen(q, k, v, cu, cu, None, (w, 0), True), q.float(),
        k.float(), v.float(), do.float())
    cud = torch.tensor(cu, dtype=torch.int32, device="cuda")
    q4, do4 = q.cuda().unsqueeze(0), do.cuda().unsqueeze(0)
    kv = torch.stack([k.cuda(), v.cuda()]).unsqueeze(1)
    acc = torch.zeros(1, total, hq, d, device="cuda")
    lacc = torch.full((1, hq, total), float("-inf"), dtype=torch.float64, device="cuda")
    flash_attn_varlen_fwd_func(q4, kv, d ** -0.5, (w, 0), cud, cud, None, None, True, acc, lacc)
    torch.cuda.synchronize()
    assert (acc[0].cpu() - ro).abs().max().item() <= 2e-2
    assert (lacc[0].float().cpu() - rl).abs().max().item() <= 1e-3
    dq, dkv = torch.empty_like(q4), torch.empty_like(kv)
    flash_attn_varlen_bwd_func(q4, kv, acc.bfloat16(), lacc.float(), do4, dq, dkv, cud, cud, None,
                               None, d ** -0.5, (w, 0), True)
    torch.cuda.synchronize()
    errs = [relnorm(dq[0], rq), relnorm(dkv[0, 0], rk), relnorm(dkv[1, 0], rv)]
    assert max(errs) <= GRAD_TOL, errs


def test_ops_namespace_has_the_upstream_names():
    import ring_swa.ops as ops

    for name in ("flash_attn_fwd_func", "flash_attn_bwd_func", "flash_attn_varlen_fwd_func",
                 "flash_attn_varlen_bwd_func", "wrapped_flash_attn_fwd", "wrapped_flash_attn_bwd",
                 "wrapped_flash_attn_fwd_varlen", "wrapped_flash_attn_bwd_varlen", "merge_attn_out",
                 "ring_attn_p2p_communicate", "get_group_local_to_global_rank_map"):
        assert callable(getattr(ops, name)), name
