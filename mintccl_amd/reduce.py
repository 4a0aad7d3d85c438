"""Ring reduce (``5_reduce.py``): elementwise sum in ring order, in place at
the root; the other ranks' buffers are left as they were.
``MINTCCL_TOPOLOGY=tree`` adds up a binary tree instead (``mintccl_amd.tree``)."""
from __future__ import annotations

import torch

from . import _lib
from ._ops import (check_buffer, comm_or_default, nbytes, reduce_dtype, ring_of,
                   same_everywhere)
from .common import VirtualComm


def reduce(buff: torch.Tensor, root: int, comm: VirtualComm | None = None) -> None:
    from . import tree
    if tree.topology_env() == "tree":
        return tree.reduce(buff, root, comm)
    comm = comm_or_default(comm)
    check_buffer(buff, comm)
    posted = comm.post("reduce", set(range(comm.world_size)),
                       {"ptr": buff.data_ptr(), "count": nbytes(buff), "root": root,
                        "dtype": reduce_dtype(buff), "keep": buff})
    if posted is None:
        return
    count = same_everywhere(posted, "count", "the byte count")
    root = same_everywhere(posted, "root", "the root")
    dtype = same_everywhere(posted, "dtype", "the dtype")
    ptrs = {r: info["ptr"] for r, info in posted.items()}
    # inputbuff on every rank, outputbuff only at the root (5_reduce.py:117-118)
    d = comm.make_op(_lib.OP_REDUCE, dtype, count, ptrs, {root: ptrs[root]}, ring_of(comm),
                     root=root)
    comm.launch(d)


if __name__ == "__main__":      # the reference runs its self-test from here
    import sys

    from .selftest import main
    sys.exit(main("reduce"))
