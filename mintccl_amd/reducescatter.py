"""Ring reduce-scatter (``7_reducescatter.py``): ``buff`` is ``(world, n)``;
after the call row r of rank r holds the sum over ranks of their row r,
accumulated in ring order starting from rank r's own value.
``MINTCCL_TOPOLOGY=hypercube`` halves recursively instead
(``mintccl_amd.hypercube``)."""
from __future__ import annotations

import torch

from . import _lib
from ._ops import (check_buffer, comm_or_default, nbytes, reduce_dtype, ring_of,
                   same_everywhere)
from .common import VirtualComm


def reducescatter(buff: torch.Tensor, comm: VirtualComm | None = None) -> None:
    from . import hypercube, tree
    if tree.topology_env() == "hypercube":
        return hypercube.reducescatter(buff, comm)
    comm = comm_or_default(comm)
    check_buffer(buff, comm)
    if buff.numel() % comm.world_size:
        raise ValueError("buffer does not split into world_size rows")
    posted = comm.post("reducescatter", set(range(comm.world_size)),
                       {"ptr": buff.data_ptr(), "count": nbytes(buff),
                        "dtype": reduce_dtype(buff), "keep": buff})
    if posted is None:
        return
    count = same_everywhere(posted, "count", "the byte count")
    dtype = same_everywhere(posted, "dtype", "the dtype")
    row = count // comm.world_size
    ptrs = {r: info["ptr"] for r, info in posted.items()}
    d = comm.make_op(_lib.OP_REDUCESCATTER, dtype, row, ptrs, ptrs, ring_of(comm),
                     row_stride=row)
    comm.launch(d)


if __name__ == "__main__":      # the reference runs its self-test from here
    import sys

    from .selftest import main
    sys.exit(main("reducescatter"))
