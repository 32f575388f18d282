"""The whole path under HIP graph capture: the library neither allocates nor synchronises,
and the rank step's second stream is forked and joined with events, so a forward +
backward step can be captured once and replayed.  Every replay (with eager work and
synchronisations in between) must reproduce the eager result bit for bit."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _inputs(seed, s, hq, hk, d=128):
    g = torch.Generator().manual_seed(seed)
    mk = lambda *shape: torch.randn(*shape, generator=g).bfloat16().cuda()  # noqa: E731
    return mk(1, s, hq, d), mk(1, s, hk, d), mk(1, s, hk, d), mk(2, 1, s, hk, d), mk(1, s, hq, d)


@pytest.mark.parametrize("w", [300, 256], ids=["two_blocks", "one_band_pass"])
def test_rank_share_step_replays_from_a_graph(w):
    import ring_swa

    s, hq, hk, cp, rank = 512, 4, 2, 4, 2
    q, k, v, prev, do = _inputs(0, s, hq, hk)
    sq, sk, sv, sprev, sdo = (torch.empty_like(t) for t in (q, k, v, prev, do))
    for dst, src in ((sq, q), (sk, k), (sv, v), (sprev, prev), (sdo, do)):
        dst.copy_(src)
    sq.requires_grad_(), sk.requires_grad_(), sv.requires_grad_(), sprev.requires_grad_()

    def step():
        out = ring_swa.ring_rank_share_attn(sq, sk, sv, [sprev], w, cp, rank)
        grads = torch.autograd.grad(out, (sq, sk, sv, sprev), sdo)
        return (out.detach(), *grads)

    # warm up on a side stream (allocator pools, lazy library state), then capture
    warm = torch.cuda.Stream()
    warm.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(warm):
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(warm)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    for trial in range(3):
        q2, k2, v2, prev2, do2 = _inputs(10 + trial, s, hq, hk)
        for dst, src in ((sq, q2), (sk, k2), (sv, v2), (sprev, prev2), (sdo, do2)):
            dst.detach().copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        eager = step()  # eager work between the replays
        torch.cuda.synchronize()
        for a, b in zip(got, eager):
            assert torch.isfinite(a.float()).all()
            assert torch.equal(a, b), f"replay {trial} differs from the eager step"
