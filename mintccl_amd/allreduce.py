"""Ring allreduce: the collective the reference lists as planned
(``8_allreduce.py``, ``README.md:23,49``), built from the pieces of
``7_reducescatter.py`` and ``6_allgather.py``: the buffer is cut into
``world`` chunks; chunk c is summed round the ring starting from rank c's own
value (the reduce-scatter order of ``7_reducescatter.py:54-73``) and the
finished sum keeps travelling until every rank has stored it.  In place; after
the call all ranks hold the same bits."""
from __future__ import annotations

import torch

from . import _lib
from ._ops import (check_buffer, comm_or_default, nbytes, reduce_dtype, ring_of,
                   same_everywhere)
from .common import VirtualComm


def allreduce(buff: torch.Tensor, comm: VirtualComm | None = None) -> None:
    comm = comm_or_default(comm)
    check_buffer(buff, comm)
    posted = comm.post("allreduce", set(range(comm.world_size)),
                       {"ptr": buff.data_ptr(), "count": nbytes(buff),
                        "dtype": reduce_dtype(buff), "keep": buff})
    if posted is None:
        return
    count = same_everywhere(posted, "count", "the byte count")
    dtype = same_everywhere(posted, "dtype", "the dtype")
    ptrs = {r: info["ptr"] for r, info in posted.items()}
    d = comm.make_op(_lib.OP_ALLREDUCE, dtype, count, ptrs, ptrs, ring_of(comm))
    comm.launch(d)


if __name__ == "__main__":      # the reference runs its self-test from here
    import sys

    from .selftest import main
    sys.exit(main("allreduce"))
