"""Host logic of the rank-share path, on CPU: the blocks a rank plans must tile
exactly the global band mask (brute force over small geometries), and the
public entry points must reject what this build does not cover."""
import pytest
import torch

from oracle import attention_oracle as O
from ring_swa import rank_share as RS


def _global_mask(total, w, cu=None):
    pos = torch.arange(total)
    sid = torch.zeros(total, dtype=torch.long) if cu is None else \
        torch.bucketize(pos, torch.tensor(cu[1:]), right=True)
    return O.global_band_allowed(pos, pos, sid, sid, w)


@pytest.mark.parametrize("seq_len,cp", [(4, 2), (4, 4), (5, 3), (7, 2)])
def test_plan_nonvarlen_tiles_global_band(seq_len, cp):
    total = seq_len * cp
    for w in range(1, total + 2):
        want = _global_mask(total, w)
        for r in range(cp):
            got = torch.zeros(seq_len, total, dtype=torch.bool)
            for (i, qs, ks, window, causal) in RS.plan_nonvarlen(seq_len, w, cp, r):
                kv0 = (r - i) * seq_len
                m = O.window_allowed(qs.stop - qs.start, ks.stop - ks.start, window, causal)
                view = got[qs, kv0 + ks.start: kv0 + ks.stop]
                assert not (view & m).any()
                view |= m
            assert torch.equal(got, want[r * seq_len:(r + 1) * seq_len]), (w, r)
        # same plan as the oracle's restatement of the reference classification
        for r in range(cp):
            assert RS.plan_nonvarlen(seq_len, w, cp, r) == O.ring_steps_nonvarlen(seq_len, w, cp, r)


def test_plan_varlen_tiles_global_band():
    g = torch.Generator().manual_seed(11)
    for _ in range(80):
        cp = int(torch.randint(2, 5, (1,), generator=g))
        seq_len = int(torch.randint(3, 8, (1,), generator=g))
        total = cp * seq_len
        ncut = int(torch.randint(0, 4, (1,), generator=g))
        cuts = sorted(set(torch.randint(1, total, (ncut,), generator=g).tolist()))
        cu = [0] + cuts + [total]
        w = int(torch.randint(1, total + 1, (1,), generator=g))
        want = _global_mask(total, w, cu)
        for r in range(cp):
            local_cu, plan = RS.plan_varlen(cu, seq_len, w, cp, r)
            assert (local_cu, plan) == O.ring_steps_varlen(cu, seq_len, w, cp, r)
            got = torch.zeros(seq_len, total, dtype=torch.bool)
            for (i, qs, ks, window, causal) in plan:
                kv0 = (r - i) * seq_len
                if i == 0:
                    for a, b in zip(local_cu[:-1], local_cu[1:]):
                        got[a:b, kv0 + a: kv0 + b] |= O.window_allowed(b - a, b - a, window, causal)
                else:
                    got[qs, kv0 + ks.start: kv0 + ks.stop] |= O.window_allowed(
                        qs.stop - qs.start, ks.stop - ks.start, window, causal)
            assert torch.equal(got, want[r * seq_len:(r + 1) * seq_len]), (cu, seq_len, w, r)


def test_benchmark_geometry():
    # virtual cp 8, chunk 8192, window 4096: one hop, upper-right 4096 x 4096 corner
    plan = RS.plan_nonvarlen(8192, 4096, 8, 3)
    assert plan == [(0, slice(0, 8192), slice(0, 8192), (4096, 0), True),
                    (1, slice(0, 4096), slice(4096, 8192), (0, 8192), False)]
    assert RS.plan_nonvarlen(8192, 4096, 8, 0) == plan[:1]  # rank 0 has no predecessor
    assert RS.ring_comm_times(4096, 8192, 8) == 1 and RS.ring_comm_times(20000, 8192, 8) == 3
    assert RS.ring_comm_times(10 ** 6, 8192, 8) == 7


def test_public_api_rejects_cpu_tensors_and_bad_arguments():
    import ring_swa

    q = torch.zeros(1, 8, 4, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU path"):
        ring_swa.ring_sliding_window_attn(q, q, q, 4)
    with pytest.raises(AssertionError):
        ring_swa.ring_sliding_window_attn(q, q[:, :4], q[:, :4], 4)
    p = torch.zeros(8, 4, 128, dtype=torch.bfloat16)
    cu = torch.tensor([0, 8], dtype=torch.int32)
    with pytest.raises(RuntimeError, match="no CPU path"):
        ring_swa.ring_streaming_llm_attn_varlen(p, p, p, 4, cu)
    with pytest.raises(ValueError):
        ring_swa.ring_streaming_llm_attn(q, q, q, 4, impl="other")


def test_signatures_match_upstream_order():
    import inspect

    import ring_swa

    base = ["q", "k", "v", "window_size"]
    cp = ["cp_group", "cp_size", "cp_local_rank", "cp_prev_global_rank", "cp_next_global_rank",
          "softmax_scale"]
    for fn, extra in ((ring_swa.ring_sliding_window_attn, []),
                      (ring_swa.ring_sliding_window_attn_varlen, ["cu_seqlens"]),
                      (ring_swa.ring_streaming_llm_attn, []),
                      (ring_swa.ring_streaming_llm_attn_varlen, ["cu_seqlens"])):
        params = [n for n, p in inspect.signature(fn).parameters.items()
                  if p.kind is p.POSITIONAL_OR_KEYWORD]
        assert params == base + extra + cp, fn.__name__
