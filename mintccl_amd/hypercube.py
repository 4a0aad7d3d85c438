"""Reduce-scatter and allgather over a hypercube of the ranks - "Hypercube" on
the reference's roadmap (``README.md:52-55``), with the argument lists and
buffers of ``7_reducescatter.py:81`` and ``6_allgather.py:141``: ``buff`` is
``(world, n)`` and row r belongs to rank r.

The cube is laid over the communicator's ring: node ``i`` is the i-th rank of
the ring, and a world of 2, 4 or 8 ranks has 1, 2 or 3 dimensions.
*Recursive halving* (reduce-scatter): in exchange ``k = 0, 1, ..`` node ``i``
and node ``i ^ (world >> (k + 1))`` split the rows they still hold - each keeps
the half its own number lies in and adds the partner's partial sums to its
own.  After ``log2(world)`` exchanges node ``i`` holds the finished row of its
rank, where the ring takes ``world - 1`` hops, which is what a small message
pays for.  The partial sum a node passes on in exchange ``k`` is

    ((own + partner 0) + partner 1) + ... + partner k-1

one rounding per addition (``order`` below spells it out per row).
*Recursive doubling* (allgather) runs the exchanges backwards: a row spreads
from its owner to the partner of the last exchange, from both to the partners
of the one before, and so on.

``MINTCCL_TOPOLOGY=hypercube`` makes ``mintccl_amd.reducescatter.reducescatter``
and ``mintccl_amd.allgather.allgather`` come here (LL128 only, world a power of
two).
"""
from __future__ import annotations

import torch

from . import _lib
from ._ops import (check_buffer, comm_or_default, nbytes, reduce_dtype, ring_of,
                   same_everywhere)
from .common import VirtualComm


def nodes(ring: list[int]) -> list[int]:
    """Ranks in node order: ``nodes[i]`` is corner ``i`` of the cube."""
    return list(ring[:-1]) if len(ring) > 1 and ring[-1] == ring[0] else list(ring)


def dimensions(world: int) -> int:
    if world < 1 or world & (world - 1):
        raise ValueError("a hypercube has 2, 4 or 8 ranks")
    return world.bit_length() - 1


def order(world: int, owner: int, node: int | None = None):
    """The additions that make row ``owner`` (a node number), as a nested
    tuple of node numbers: ``((own, a), b)`` = (own + a) + b, where ``a`` and
    ``b`` are such tuples themselves."""
    dim = dimensions(world)
    node = owner if node is None else node
    split = next((k for k in range(dim) if (node ^ owner) & (1 << (dim - 1 - k))), dim)
    acc = node
    for k in range(split):
        acc = (acc, order(world, owner, node ^ (1 << (dim - 1 - k))))
    return acc


def _check_world(comm: VirtualComm) -> None:
    dimensions(comm.world_size)


def reducescatter(buff: torch.Tensor, comm: VirtualComm | None = None) -> None:
    comm = comm_or_default(comm)
    _check_world(comm)
    check_buffer(buff, comm)
    if buff.numel() % comm.world_size:
        raise ValueError("buffer does not split into world_size rows")
    posted = comm.post("hypercube_reducescatter", set(range(comm.world_size)),
                       {"ptr": buff.data_ptr(), "count": nbytes(buff),
                        "dtype": reduce_dtype(buff), "keep": buff})
    if posted is None:
        return
    count = same_everywhere(posted, "count", "the byte count")
    dtype = same_everywhere(posted, "dtype", "the dtype")
    row = count // comm.world_size
    ptrs = {r: info["ptr"] for r, info in posted.items()}
    d = comm.make_op(_lib.OP_HYPERCUBE_REDUCESCATTER, dtype, row, ptrs, ptrs, ring_of(comm),
                     row_stride=row, protocol=_lib.PROTO_LL128)
    comm.launch(d)


def allgather(buff: torch.Tensor, comm: VirtualComm | None = None) -> None:
    comm = comm_or_default(comm)
    _check_world(comm)
    check_buffer(buff, comm)
    if nbytes(buff) % comm.world_size:
        raise ValueError("buffer does not split into world_size rows")
    posted = comm.post("hypercube_allgather", set(range(comm.world_size)),
                       {"ptr": buff.data_ptr(), "count": nbytes(buff), "keep": buff})
    if posted is None:
        return
    count = same_everywhere(posted, "count", "the byte count")
    row = count // comm.world_size
    ptrs = {r: info["ptr"] for r, info in posted.items()}
    d = comm.make_op(_lib.OP_HYPERCUBE_ALLGATHER, _lib.BYTES, row, ptrs, ptrs, ring_of(comm),
                     row_stride=row, protocol=_lib.PROTO_LL128)
    comm.launch(d)


if __name__ == "__main__":      # self-test in the reference's style: both collectives
    import sys

    from .selftest import main
    sys.exit(max(main("hypercube_reducescatter"), main("hypercube_allgather")))
