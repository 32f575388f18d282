"""Point-to-point exchange of KV / dKV chunks between context-parallel ranks, and the
group-local -> global rank map.

Takes the place of ``ring_swa/ops/comm.py:8-40`` (``ring_attn_p2p_communicate``) and
``:152-232`` (``get_group_local_to_global_rank_map``) of the upstream package.  Works on any
``torch.distributed`` backend: ``"nccl"`` (RCCL over xGMI on MI355X nodes) with device
tensors, ``"gloo"`` with host tensors (the CPU test tier of the ring logic).

On an MI355X node every GPU has a direct xGMI link to every other, so a rank that needs the
chunks of several predecessors fetches them from their owners at once, each over its own
link, instead of relaying one chunk per hop around a ring: ``exchange`` posts all sends and
receives of a phase as one batch.
"""
from __future__ import annotations

from typing import Dict, List, Sequence, Tuple

import torch
import torch.distributed as dist


def get_group_local_to_global_rank_map(group) -> Dict[int, int]:
    """``{rank inside the group: global rank}`` for ``group`` (``{}`` for ``None``).

    The group already knows its members in group order, so no collective is needed
    (upstream gathers ``(local, global)`` pairs with an all-gather, ``ops/comm.py:185-208``)
    and the call is safe from any subset of the ranks."""
    if group is None:
        return {}
    return dict(enumerate(dist.get_process_group_ranks(group)))


class _StagedWork:
    """Requests of a batch whose device tensors travel through host memory: ``wait`` completes
    the transfers and copies what was received into the device buffers."""

    def __init__(self, works, landed):
        self._works, self._landed = works, landed

    def wait(self):
        for w in self._works:
            w.wait()
        for buf, host in self._landed:
            buf.copy_(host)
        self._landed = []


def exchange(sends: Sequence[Tuple[torch.Tensor, int]], recvs: Sequence[Tuple[torch.Tensor, int]],
             group) -> List["dist.Work"]:
    """Post every ``(tensor, global destination)`` send and ``(buffer, global source)``
    receive of one phase as a single batch; returns the requests to wait on.  Tensors must be
    contiguous; an empty phase returns no requests.

    A gloo group takes host tensors only: device tensors are staged through host memory
    (synchronous copy out before the send, copy back in ``wait``) -- the route for rehearsing
    the ring with several processes on one GPU; RCCL groups get the device tensors as they are."""
    if not sends and not recvs:
        return []
    on_device = any(t.is_cuda for t, _ in list(sends) + list(recvs))
    if on_device and dist.get_backend(group) == "gloo":
        landed = [(buf, torch.empty(buf.shape, dtype=buf.dtype)) for buf, _ in recvs]
        ops = [dist.P2POp(dist.irecv, host, src, group) for (_, host), (_, src) in zip(landed, recvs)]
        ops += [dist.P2POp(dist.isend, t.cpu(), dst, group) for t, dst in sends]
        return [_StagedWork(dist.batch_isend_irecv(ops), landed)]
    ops = [dist.P2POp(dist.irecv, buf, src, group) for buf, src in recvs]
    ops += [dist.P2POp(dist.isend, t, dst, group) for t, dst in sends]
    return dist.batch_isend_irecv(ops)


def ring_attn_p2p_communicate(rank: int, send_tensor: torch.Tensor, send_rank: int,
                              recv_tensor: torch.Tensor, recv_rank: int, cp_group) -> List["dist.Work"]:
    """One send and one receive between ring neighbours, upstream's signature
    (``ops/comm.py:8-40``; ``rank`` ordered its sends and receives by parity to avoid a
    deadlock, which the batched form does not need)."""
    return exchange([(send_tensor, send_rank)], [(recv_tensor, recv_rank)], cp_group)
