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


def exchange(sends: Sequence[Tuple[torch.Tensor, int]], recvs: Sequence[Tuple[torch.Tensor, int]],
             group) -> List["dist.Work"]:
    """Post every ``(tensor, global destination)`` send and ``(buffer, global source)``
    receive of one phase as a single batch; returns the requests to wait on.  Tensors must be
    contiguous; an empty phase returns no requests."""
    ops = [dist.P2POp(dist.irecv, buf, src, group) for buf, src in recvs]
    ops += [dist.P2POp(dist.isend, t, dst, group) for t, dst in sends]
    if not ops:
        return []
    return dist.batch_isend_irecv(ops)


def ring_attn_p2p_communicate(rank: int, send_tensor: torch.Tensor, send_rank: int,
                              recv_tensor: torch.Tensor, recv_rank: int, cp_group) -> List["dist.Work"]:
    """One send and one receive between ring neighbours, upstream's signature
    (``ops/comm.py:8-40``; ``rank`` ordered its sends and receives by parity to avoid a
    deadlock, which the batched form does not need)."""
    return exchange([(send_tensor, send_rank)], [(recv_tensor, recv_rank)], cp_group)
