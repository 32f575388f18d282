"""Point-to-point exchange of KV / dKV chunks between context-parallel ranks, and the
group-local -> global rank map.

Takes the place of ``ring_swa/ops/comm.py:8-40`` (``ring_attn_p2p_communicate``),
``:43-149`` (``broadcast_tensor_to_group``, ``reduce_sum_tesnsor_to_rank``,
``exchange_and_sum_tensors``: the helpers of upstream's streaming-LLM ring, kept under their
names -- the ring of this package moves its sink rows point to point and does not call them)
and ``:152-232`` (``get_group_local_to_global_rank_map``) of the upstream package.  Works on any
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


class _StagedCollective:
    """Work handle of a collective on a gloo group whose tensor lives on a device: the data
    travelled in a host copy, ``wait`` completes the collective and, where the rank receives,
    copies the result back."""

    def __init__(self, work, tensor, host, receives):
        self._work, self._tensor, self._host, self._receives = work, tensor, host, receives

    def wait(self):
        self._work.wait()
        if self._receives and self._host is not None:
            self._tensor.copy_(self._host)
            self._host = None
        return True


def _staged(tensor: torch.Tensor, group):
    """``(tensor the collective runs on, needs copy-back)``: gloo takes host tensors only."""
    if tensor.is_cuda and dist.get_backend(group) == "gloo":
        return tensor.cpu(), True
    return tensor, False


def broadcast_tensor_to_group(tensor: torch.Tensor, src_rank: int, cp_group):
    """Asynchronous broadcast of ``tensor`` from global rank ``src_rank`` to every rank of
    ``cp_group`` (``ops/comm.py:43-70``): returns a handle whose ``wait()`` completes it.
    Every rank of the group calls it with a tensor of the same shape and dtype."""
    host, staged = _staged(tensor, cp_group)
    work = dist.broadcast(host, src=src_rank, group=cp_group, async_op=True)
    if not staged:
        return work
    return _StagedCollective(work, tensor, host, dist.get_rank() != src_rank)


def reduce_sum_tesnsor_to_rank(tensor: torch.Tensor, dst_rank: int, cp_group) -> torch.Tensor:
    """Sum of every rank's ``tensor`` on global rank ``dst_rank``, in place (``ops/comm.py:73-100``,
    upstream's spelling of the name); blocking; returns ``tensor`` (on the other ranks its
    contents are unspecified afterwards, as with ``dist.reduce``)."""
    host, staged = _staged(tensor, cp_group)
    dist.reduce(host, dst=dst_rank, op=dist.ReduceOp.SUM, group=cp_group)
    if staged and dist.get_rank() == dst_rank:
        tensor.copy_(host)
    return tensor


def exchange_and_sum_tensors(tensor_to_send: torch.Tensor, send_to_rank: int, cp_group) -> torch.Tensor:
    """Every rank sends its tensor to ONE rank of its choice (group-local index
    ``send_to_rank``, as upstream's all-to-all slot, ``ops/comm.py:103-149``); returns the sum of
    what this rank received (zeros if nobody sent to it).  Blocking; same shape and dtype on
    every rank.

    Upstream fills an all-to-all with a zero tensor for every rank that is not the destination
    (world size times the payload in flight).  Here the ranks first share their destinations (one
    integer each), then only the real payloads travel, point to point; they are added in rank
    order, so the sum does not depend on arrival order."""
    world = dist.get_world_size(group=cp_group)
    me = dist.get_rank(group=cp_group)
    members = dist.get_process_group_ranks(cp_group)
    dests = [torch.zeros(1, dtype=torch.int64) for _ in range(world)]
    mine = torch.tensor([int(send_to_rank)], dtype=torch.int64)
    if dist.get_backend(cp_group) != "gloo":
        mine = mine.to(tensor_to_send.device)
        dests = [d.to(tensor_to_send.device) for d in dests]
    dist.all_gather(dests, mine, group=cp_group)
    dests = [int(d.item()) for d in dests]
    senders = [r for r in range(world) if dests[r] == me and r != me]
    bufs = [torch.empty_like(tensor_to_send) for _ in senders]
    sends = [] if dests[me] == me else [(tensor_to_send.contiguous(), members[dests[me]])]
    for w in exchange(sends, [(b, members[r]) for b, r in zip(bufs, senders)], cp_group):
        w.wait()
    total = torch.zeros_like(tensor_to_send)
    parts = dict(zip(senders, bufs))
    if dests[me] == me:
        parts[me] = tensor_to_send
    for r in sorted(parts):
        total += parts[r]
    return total
