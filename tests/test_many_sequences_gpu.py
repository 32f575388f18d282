"""Packs of hundreds and thousands of short sequences: every block has to find its sequence
among them (a search over cu_seqlens inside the kernels), sequences shorter than one tile
leave tile slots unused, and several sequences share one 128- or 256-row stretch of the pack."""
import pytest
import torch

from oracle import attention_oracle as O
from tests.gradcheck_util import GRAD_TOL, relnorm

pytestmark = pytest.mark.gpu


def _pack(n_seq, lo, hi, seed):
    g = torch.Generator().manual_seed(seed)
    lens = torch.randint(lo, hi + 1, (n_seq,), generator=g).tolist()
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    return cu


@pytest.mark.parametrize("n_seq,lo,hi,window,sink,d", [
    (640, 1, 48, 16, 0, 128),
    (513, 1, 40, 8, 2, 64),
    (700, 1, 3, 1, 0, 128),      # hundreds of sequences inside one tile
], ids=["640x1-48", "513x1-40_sinks", "700x1-3"])
def test_pack_of_many_short_sequences(n_seq, lo, hi, window, sink, d):
    from ring_swa.ops import attn_bwd, attn_fwd

    cu = _pack(n_seq, lo, hi, seed=n_seq)
    t, hq, hk = cu[-1], 2, 1
    torch.manual_seed(n_seq)
    q, do = (torch.randn(t, hq, d, device="cuda").bfloat16() for _ in range(2))
    k, v = (torch.randn(t, hk, d, device="cuda").bfloat16() for _ in range(2))
    cu_dev = torch.tensor(cu, dtype=torch.int32, device="cuda")
    out, lse = attn_fwd(q, k, v, None, (window, 0), True, cu_dev, cu_dev, num_sink=sink)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    attn_bwd(q, k, v, out, lse, do, dq, dk, dv, None, (window, 0), True, cu_dev, cu_dev,
             num_sink=sink)
    if sink:
        fn = lambda q, k, v: O.streaming_llm_attn_varlen(q, k, v, window, cu, n_sink=sink)  # noqa: E731
    else:
        fn = lambda q, k, v: O.sliding_window_attn_varlen(q, k, v, window, cu)  # noqa: E731
    ro, rl, rq, rk, rv = O.attention_fwd_bwd(fn, q, k, v, do)
    assert (out.float() - ro).abs().max().item() <= 2e-2
    assert (lse - rl).abs().max().item() <= 1e-3
    for name, x, r in (("dq", dq, rq), ("dk", dk, rk), ("dv", dv, rv)):
        assert relnorm(x, r) <= GRAD_TOL, name


def test_pack_of_4096_sequences_equals_its_dense_view():
    """65 536 tokens as 4096 sequences of 16 (every block has to find its sequence among 4096)
    against the same problem as a dense [4096, 16] batch: the same bits.  (The time of this
    pack is a key of the benchmark, not an assertion here.)"""
    from ring_swa.ops import attn_bwd, attn_fwd

    n, L, hq, hk, d = 4096, 16, 8, 2, 128
    cu_dev = torch.arange(0, (n + 1) * L, L, dtype=torch.int32, device="cuda")
    q, do = (torch.randn(n * L, hq, d, device="cuda").bfloat16() for _ in range(2))
    k, v = (torch.randn(n * L, hk, d, device="cuda").bfloat16() for _ in range(2))
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)

    def run():
        out, lse = attn_fwd(q, k, v, None, (8, 0), True, cu_dev, cu_dev)
        attn_bwd(q, k, v, out, lse, do, dq, dk, dv, None, (8, 0), True, cu_dev, cu_dev)
        return out

    out = run()
    torch.cuda.synchronize()
    # dense view of the same problem: [4096, 16] batches
    ref, _ = attn_fwd(q.view(n, L, hq, d), k.view(n, L, hk, d), v.view(n, L, hk, d), None, (8, 0),
                      True)
    assert torch.equal(out.view(n, L, hq, d), ref)
