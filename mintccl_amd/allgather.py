"""Ring allgather (``6_allgather.py``): ``buff`` is ``(world, n)``; rank r
contributes row r and ends up with every rank's row, in place."""
from __future__ import annotations

import torch

from . import _lib
from ._ops import check_buffer, comm_or_default, nbytes, ring_of, same_everywhere
from .common import VirtualComm


def allgather(buff: torch.Tensor, comm: VirtualComm | None = None) -> None:
    comm = comm_or_default(comm)
    check_buffer(buff, comm)
    if nbytes(buff) % comm.world_size:
        raise ValueError("buffer does not split into world_size rows")
    posted = comm.post("allgather", set(range(comm.world_size)),
                       {"ptr": buff.data_ptr(), "count": nbytes(buff), "keep": buff})
    if posted is None:
        return
    count = same_everywhere(posted, "count", "the byte count")
    row = count // comm.world_size
    ptrs = {r: info["ptr"] for r, info in posted.items()}
    d = comm.make_op(_lib.OP_ALLGATHER, _lib.BYTES, row, ptrs, ptrs, ring_of(comm),
                     row_stride=row)
    comm.launch(d)


if __name__ == "__main__":      # the reference runs its self-test from here
    import sys

    from .selftest import main
    sys.exit(main("allgather"))
