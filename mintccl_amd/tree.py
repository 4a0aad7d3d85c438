"""Broadcast and reduce over a binary tree of the ranks - "Tree / Binary Tree"
on the reference's roadmap (``README.md:52-55``), with the argument lists of
``4_broadcast.py:79`` and ``5_reduce.py:99``.

The tree is laid over the communicator's ring, turned so that the root comes
first: node ``h`` (0 = root) has parent ``(h - 1) // 2`` and children
``2h + 1``, ``2h + 2``.  Eight ranks are three hops deep where the ring is
seven, which is what a small message pays for.  A node of a reduce passes up
``(own + first subtree) + second subtree``, one rounding per addition.

``MINTCCL_TOPOLOGY=tree`` makes ``mintccl_amd.broadcast.broadcast`` and
``mintccl_amd.reduce.reduce`` come here.
"""
from __future__ import annotations

import os

import torch

from . import _lib
from ._ops import (check_buffer, comm_or_default, nbytes, reduce_dtype, ring_of,
                   same_everywhere)
from .common import VirtualComm


def topology_env() -> str:
    return os.getenv("MINTCCL_TOPOLOGY", "ring").lower()


def nodes(ring: list[int], root: int) -> list[int]:
    """Ranks in node order: ``nodes[h]`` is node ``h`` of the tree."""
    order = list(ring[:-1]) if len(ring) > 1 and ring[-1] == ring[0] else list(ring)
    at = order.index(root)
    return order[at:] + order[:at]


def broadcast(buff: torch.Tensor, root: int, comm: VirtualComm | None = None) -> None:
    comm = comm_or_default(comm)
    check_buffer(buff, comm)
    posted = comm.post("tree_broadcast", set(range(comm.world_size)),
                       {"ptr": buff.data_ptr(), "count": nbytes(buff), "root": root, "keep": buff})
    if posted is None:
        return
    count = same_everywhere(posted, "count", "the byte count")
    root = same_everywhere(posted, "root", "the root")
    ptrs = {r: info["ptr"] for r, info in posted.items()}
    d = comm.make_op(_lib.OP_TREE_BROADCAST, _lib.BYTES, count, {root: ptrs[root]},
                     {r: p for r, p in ptrs.items() if r != root}, ring_of(comm), root=root,
                     protocol=_lib.PROTO_LL128)
    comm.launch(d)


def reduce(buff: torch.Tensor, root: int, comm: VirtualComm | None = None) -> None:
    comm = comm_or_default(comm)
    check_buffer(buff, comm)
    posted = comm.post("tree_reduce", set(range(comm.world_size)),
                       {"ptr": buff.data_ptr(), "count": nbytes(buff), "root": root,
                        "dtype": reduce_dtype(buff), "keep": buff})
    if posted is None:
        return
    count = same_everywhere(posted, "count", "the byte count")
    root = same_everywhere(posted, "root", "the root")
    dtype = same_everywhere(posted, "dtype", "the dtype")
    ptrs = {r: info["ptr"] for r, info in posted.items()}
    d = comm.make_op(_lib.OP_TREE_REDUCE, dtype, count, ptrs, {root: ptrs[root]}, ring_of(comm),
                     root=root, protocol=_lib.PROTO_LL128)
    comm.launch(d)


if __name__ == "__main__":      # self-test in the reference's style: both collectives
    import sys

    from .selftest import main
    sys.exit(max(main("tree_broadcast"), main("tree_reduce")))
