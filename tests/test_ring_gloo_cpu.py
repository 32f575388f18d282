"""The context-parallel ring (``ring_swa/ring.py``, ``cp_group`` given) on the CPU: several
processes over gloo, CPU tensors, the oracle standing in for the HIP kernels (the test hands
the stand-ins in; the package never imports the oracle).  Checks the host logic that one GPU
cannot: who sends which key range to whom, block order, dKV going back to its owner -- the
concatenation of the ranks' outputs and gradients must equal the single-call oracle on the
whole sequence, for windows shorter than a chunk, spanning several chunks and longer than the
sequence, dense and packed.  Also the group-local -> global rank map on a sub-group."""
import os
import socket
import sys
from types import SimpleNamespace

import pytest
import torch
import torch.distributed as dist
import torch.multiprocessing as mp

from oracle import attention_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _free_port():
    with socket.socket() as s:
        s.bind(("127.0.0.1", 0))
        return s.getsockname()[1]


def oracle_kernels(dtype=torch.float64):
    """The five primitives of ``ops/accum.py`` on the oracle (CPU, fp64)."""

    def fwd(q, k, v, scale, window, causal, mask_shift=None):
        return O.window_attention(q, k, v, scale, window, causal, compute_dtype=dtype,
                                  shift=mask_shift)

    def fwd_varlen(q, k, v, scale, window, cu_q, cu_k, max_q, max_k, causal):
        return O.window_attention_varlen(q, k, v, cu_q.tolist(), cu_k.tolist(), scale, window,
                                         causal, compute_dtype=dtype)

    def bwd(q, k, v, o, lse, do, dq, dk, dv, scale, window, causal, mask_shift=None):
        allowed = O.window_allowed(q.shape[1], k.shape[1], window, causal, shift=mask_shift)
        a, b, c = O.attention_bwd_from_stats(q, k, v, o, lse, do, allowed, scale, dtype)
        dq.copy_(a), dk.copy_(b), dv.copy_(c)

    def bwd_varlen(q, k, v, o, lse, do, dq, dk, dv, scale, window, cu_q, cu_k, max_q, max_k,
                   causal):
        cq, ck = cu_q.tolist(), cu_k.tolist()
        for a0, a1, b0, b1 in zip(cq[:-1], cq[1:], ck[:-1], ck[1:]):
            if a1 == a0:
                continue
            allowed = O.window_allowed(a1 - a0, b1 - b0, window, causal)
            a, b, c = O.attention_bwd_from_stats(
                q[None, a0:a1], k[None, b0:b1], v[None, b0:b1], o[None, a0:a1], lse[None, :, a0:a1],
                do[None, a0:a1], allowed, scale, dtype)
            dq[a0:a1], dk[b0:b1], dv[b0:b1] = a[0], b[0], c[0]

    def merge(o, lse, o_new, lse_new):
        om, lm = O.merge(o.double(), lse.double(), o_new.double(), lse_new.double())
        o.copy_(om), lse.copy_(lm)

    return SimpleNamespace(fwd=fwd, fwd_varlen=fwd_varlen, bwd=bwd, bwd_varlen=bwd_varlen,
                           merge=merge)


def _check_collective_helpers(rank, world, group):
    """The three helpers of upstream's streaming-LLM ring (``ops/comm.py:43-149``), by their
    defining sums: broadcast copies the source's tensor, reduce leaves the sum of all on the
    destination, the exchange returns the sum of what the ranks that chose this rank sent."""
    from ring_swa.ops import (broadcast_tensor_to_group, exchange_and_sum_tensors,
                              reduce_sum_tesnsor_to_rank)

    base = torch.arange(6, dtype=torch.float64).reshape(2, 3)
    t = base * (rank + 1)
    broadcast_tensor_to_group(t, world - 1, group).wait()
    assert torch.equal(t, base * world)
    t = base + rank
    out = reduce_sum_tesnsor_to_rank(t, 0, group)
    if rank == 0:
        assert out is t and torch.equal(t, base * world + sum(range(world)))
    # everybody sends to rank 0 except rank 0, which sends to the last rank
    dest = world - 1 if rank == 0 else 0
    got = exchange_and_sum_tensors(base * 10 ** rank, dest, group)
    if rank == 0:
        want = base * sum(10 ** r for r in range(1, world))
    elif rank == world - 1:
        want = base * 1
    else:
        want = torch.zeros_like(base)
    assert torch.equal(got, want), (rank, got, want)
    # a rank may send to itself; ranks nobody sends to get zeros
    got = exchange_and_sum_tensors(base + rank, rank if rank % 2 == 0 else rank - 1, group)
    want = torch.zeros_like(base)
    if rank % 2 == 0:
        want = (base + rank) + ((base + rank + 1) if rank + 1 < world else 0)
    assert torch.equal(got, want), (rank, got, want)


def _worker(rank, world, port, cases, results):
    sys.path.insert(0, ROOT)
    sys.path.insert(0, os.path.join(ROOT, "ring-sliding-window-attention_amd"))
    dist.init_process_group("gloo", init_method=f"tcp://127.0.0.1:{port}", rank=rank,
                            world_size=world)
    torch.set_num_threads(1)
    from ring_swa.ops import get_group_local_to_global_rank_map
    from ring_swa.ring import ring_attn

    group = dist.new_group(list(range(world)))
    assert get_group_local_to_global_rank_map(group) == {i: i for i in range(world)}
    assert get_group_local_to_global_rank_map(None) == {}
    if world >= 3:
        # a sub-group whose local order differs from the global numbering
        members = [world - 1, 0]
        sub = dist.new_group(members)
        if rank in members:
            got = get_group_local_to_global_rank_map(sub)
            assert got == dict(enumerate(sorted(members))) or got == dict(enumerate(members)), got
            assert got[dist.get_rank(sub)] == rank
    _check_collective_helpers(rank, world, group)
    from ring_swa.ring_slm import ring_slm_attn

    K = oracle_kernels()
    out = {}
    for name, (q, k, v, do, w, cu, *sinks) in cases.items():
        s = q.shape[-3] // world
        sl = slice(rank * s, (rank + 1) * s)
        if sinks:
            run = lambda a, b, c, cu_: ring_slm_attn(a, b, c, w, group, world, rank, None, cu_,  # noqa: E731
                                                     num_sink_tokens=sinks[0], kernels=K)
        else:
            run = lambda a, b, c, cu_: ring_attn(a, b, c, w, group, world, rank, None, cu_,  # noqa: E731
                                                 kernels=K)
        if cu is None:
            qr, kr, vr = (t[:, sl].clone().requires_grad_() for t in (q, k, v))
            o = run(qr, kr, vr, None)
            o.backward(do[:, sl])
        else:
            qr, kr, vr = (t[sl].clone().requires_grad_() for t in (q, k, v))
            o = run(qr, kr, vr, cu)
            o.backward(do[sl])
        out[name] = (o.detach(), qr.grad, kr.grad, vr.grad)
    results[rank] = out
    dist.barrier()
    dist.destroy_process_group()


def _cases(world):
    g = torch.Generator().manual_seed(world)
    s, hq, hk, d = 6, 4, 2, 8
    total = s * world
    cases = {}
    for w in (0, 2, s - 1, s, s + 1, 2 * s - 1, 2 * s, 2 * s + 3, 10 * total):
        q, do = (torch.randn(2, total, hq, d, generator=g, dtype=torch.float64) for _ in range(2))
        k, v = (torch.randn(2, total, hk, d, generator=g, dtype=torch.float64) for _ in range(2))
        cases[f"dense_w{w}"] = (q, k, v, do, w, None)
    for n, (w, cuts) in enumerate(((3, [1, 7]), (2 * s + 1, [total - 2]), (s, [s, s + 1]),
                                   (4 * s, []), (5, list(range(2, total, 5))))):
        cu = [0] + [c for c in cuts if 0 < c < total] + [total]
        q, do = (torch.randn(total, hq, d, generator=g, dtype=torch.float64) for _ in range(2))
        k, v = (torch.randn(total, hk, d, generator=g, dtype=torch.float64) for _ in range(2))
        cases[f"packed{n}_w{w}"] = (q, k, v, do, w, cu)
    # streaming-LLM: sinks of one sequence spread over ranks, more sinks than a chunk holds,
    # windows shorter and longer than a chunk; packs whose sequences start anywhere
    for n_sink, w in ((1, 2), (3, s - 1), (2, s + 2), (s + 2, 1), (4, 3 * s), (0, 3)):
        q, do = (torch.randn(2, total, hq, d, generator=g, dtype=torch.float64) for _ in range(2))
        k, v = (torch.randn(2, total, hk, d, generator=g, dtype=torch.float64) for _ in range(2))
        cases[f"slm_dense_n{n_sink}_w{w}"] = (q, k, v, do, w, None, n_sink)
    for n, (n_sink, w, cuts) in enumerate(((1, 2, [1, 7]), (3, 1, [s - 1]), (2, s, [s, s + 1]),
                                           (4, 2, []), (2, 3, list(range(2, total, 5))),
                                           (5, 0, [s - 2, 2 * s - 1]))):
        cu = [0] + [c for c in cuts if 0 < c < total] + [total]
        q, do = (torch.randn(total, hq, d, generator=g, dtype=torch.float64) for _ in range(2))
        k, v = (torch.randn(total, hk, d, generator=g, dtype=torch.float64) for _ in range(2))
        cases[f"slm_packed{n}_n{n_sink}_w{w}"] = (q, k, v, do, w, cu, n_sink)
    return cases


@pytest.mark.parametrize("world", [2, 4])
def test_ring_over_gloo_equals_the_whole_sequence_oracle(world):
    cases = _cases(world)
    port = _free_port()
    with mp.Manager() as manager:
        results = manager.dict()
        mp.spawn(_worker, args=(world, port, cases, results), nprocs=world, join=True)
        results = dict(results)
    for name, (q, k, v, do, w, cu, *sinks) in cases.items():
        n_sink = sinks[0] if sinks else 0
        if cu is None:
            fn = lambda q, k, v: O.streaming_llm_attn(q, k, v, w, n_sink=n_sink,  # noqa: E731
                                                      compute_dtype=torch.float64)
            cat = 1
        else:
            fn = lambda q, k, v: O.streaming_llm_attn_varlen(q, k, v, w, cu, n_sink=n_sink,  # noqa: E731
                                                             compute_dtype=torch.float64)
            cat = 0
        ro, _, rq, rk, rv = O.attention_fwd_bwd(fn, q, k, v, do)
        for idx, ref in enumerate((ro, rq, rk, rv)):
            got = torch.cat([results[r][name][idx] for r in range(world)], dim=cat)
            # the saved LSE is fp32 (as upstream keeps it), which bounds the agreement of the gradients
            torch.testing.assert_close(got, ref, atol=2e-6, rtol=2e-6, msg=lambda m: f"{name}[{idx}]: {m}")
