"""Ring broadcast (``4_broadcast.py``): after the call every rank's ``buff``
holds the root's bytes.  ``MINTCCL_TOPOLOGY=tree`` sends them down a binary tree
instead (``mintccl_amd.tree``)."""
from __future__ import annotations

import torch

from . import _lib
from ._ops import check_buffer, comm_or_default, nbytes, ring_of, same_everywhere
from .common import VirtualComm


def broadcast(buff: torch.Tensor, root: int, comm: VirtualComm | None = None) -> None:
    from . import tree
    if tree.topology_env() == "tree":
        return tree.broadcast(buff, root, comm)
    comm = comm_or_default(comm)
    check_buffer(buff, comm)
    posted = comm.post("broadcast", set(range(comm.world_size)),
                       {"ptr": buff.data_ptr(), "count": nbytes(buff), "root": root, "keep": buff})
    if posted is None:
        return
    count = same_everywhere(posted, "count", "the byte count")
    root = same_everywhere(posted, "root", "the root")
    ptrs = {r: info["ptr"] for r, info in posted.items()}
    # root has the input, everyone else an output (4_broadcast.py:97-98)
    d = comm.make_op(_lib.OP_BROADCAST, _lib.BYTES, count, {root: ptrs[root]},
                     {r: p for r, p in ptrs.items() if r != root}, ring_of(comm), root=root)
    comm.launch(d)


if __name__ == "__main__":      # the reference runs its self-test from here
    import sys

    from .selftest import main
    sys.exit(main("broadcast"))
