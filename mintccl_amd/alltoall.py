"""Alltoall (the reference plans it as ``9_alltoall.py``, ``README.md:24,50``):
``buff`` and ``out`` are ``(world, n)``; after the call row ``s`` of rank
``d``'s ``out`` holds row ``d`` of rank ``s``'s ``buff`` - the transpose of the
ranks' buffers, MPI_Alltoall.  Every row travels straight to its destination
through the destination's staging slots as LL128 lines (or with the Simple
protocol): ``world x world`` pipelines of two positions in one fused launch.
``out`` must not overlap any rank's ``buff``: every row is read while others
are being written."""
from __future__ import annotations

import torch

from . import _lib
from ._ops import check_buffer, comm_or_default, nbytes, ring_of, same_everywhere
from .common import VirtualComm


def alltoall(buff: torch.Tensor, out: torch.Tensor, comm: VirtualComm | None = None) -> None:
    comm = comm_or_default(comm)
    check_buffer(buff, comm)
    check_buffer(out, comm)
    if buff.numel() % comm.world_size:
        raise ValueError("buffer does not split into world_size rows")
    if nbytes(buff) != nbytes(out):
        raise ValueError("buff and out differ in size")
    posted = comm.post("alltoall", set(range(comm.world_size)),
                       {"in": buff.data_ptr(), "out": out.data_ptr(), "count": nbytes(buff),
                        "keep": (buff, out)})
    if posted is None:
        return
    count = same_everywhere(posted, "count", "the byte count")
    row = count // comm.world_size
    lo = {r: info["in"] for r, info in posted.items()}
    for a in posted.values():
        for b in posted.values():
            if a["in"] < b["out"] + count and b["out"] < a["in"] + count:
                raise ValueError("alltoall: out overlaps a rank's buff")
    d = comm.make_op(_lib.OP_ALLTOALL, _lib.BYTES, row, lo,
                     {r: info["out"] for r, info in posted.items()}, ring_of(comm),
                     row_stride=row)
    comm.launch(d)


if __name__ == "__main__":      # the reference runs its self-test from here
    import sys

    from .selftest import main
    sys.exit(main("alltoall"))
