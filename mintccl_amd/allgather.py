"""Ring allgather (``6_allgather.py``): ``buff`` is ``(world, n)``; rank r
contributes row r and ends up with every rank's row, in place.

The reference has two kernels that leave the same bytes.  *Spatial*
(``6_allgather.py:79-138``): every source rank's row has its own blocks and
its own share of the staging - the default here, it is the faster one.
*Temporal* (``:25-77``, the one the reference's host function launches): the
whole grid moves rank 0's row round the ring, then rank 1's, and so on,
through staging for one row - ``schedule="temporal"`` or
``MINTCCL_ALLGATHER=temporal`` (LL128 only).  ``MINTCCL_TOPOLOGY=hypercube``
doubles recursively over a hypercube instead (``mintccl_amd.hypercube``)."""
from __future__ import annotations

import os

import torch

from . import _lib
from ._ops import check_buffer, comm_or_default, nbytes, ring_of, same_everywhere
from .common import VirtualComm


def allgather(buff: torch.Tensor, comm: VirtualComm | None = None,
              schedule: str | None = None) -> None:
    from . import hypercube, tree
    if schedule is None and tree.topology_env() == "hypercube":
        return hypercube.allgather(buff, comm)
    if schedule is None:
        schedule = os.getenv("MINTCCL_ALLGATHER", "spatial").lower()
    if schedule not in ("spatial", "temporal"):
        raise ValueError("allgather schedule is 'spatial' or 'temporal'")
    comm = comm_or_default(comm)
    check_buffer(buff, comm)
    if nbytes(buff) % comm.world_size:
        raise ValueError("buffer does not split into world_size rows")
    posted = comm.post("allgather", set(range(comm.world_size)),
                       {"ptr": buff.data_ptr(), "count": nbytes(buff), "schedule": schedule,
                        "keep": buff})
    if posted is None:
        return
    count = same_everywhere(posted, "count", "the byte count")
    row = count // comm.world_size
    ptrs = {r: info["ptr"] for r, info in posted.items()}
    if same_everywhere(posted, "schedule", "the schedule") == "temporal":
        d = comm.make_op(_lib.OP_ALLGATHER_TEMPORAL, _lib.BYTES, row, ptrs, ptrs, ring_of(comm),
                         row_stride=row, protocol=_lib.PROTO_LL128)
    else:
        d = comm.make_op(_lib.OP_ALLGATHER, _lib.BYTES, row, ptrs, ptrs, ring_of(comm),
                         row_stride=row)
    comm.launch(d)


if __name__ == "__main__":      # the reference runs its self-test from here
    import sys

    from .selftest import main
    sys.exit(main("allgather"))
