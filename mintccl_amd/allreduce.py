"""Ring allreduce: the collective the reference lists as planned
(``8_allreduce.py``, ``README.md:23,49``), built from the pieces of
``7_reducescatter.py`` and ``6_allgather.py``: the buffer is cut into
``world`` chunks of whole 16-byte vectors (the last ones may be short or
empty); chunk c is summed round the ring starting from rank c's own value
(the reduce-scatter order of ``7_reducescatter.py:54-73``) and the finished sum
is handed round until every rank has stored it.  In place; after the call all
ranks hold the same bits.

Two ways to run it, same result bit for bit:

* fused (``fused=True`` or ``MINTCCL_ALLREDUCE=fused``; the default below
  32 MiB per rank): one launch, one pass round the ring of 2 * world - 1
  positions - what the reference plans.  Its two phases share the staging
  slots and the wavefronts.
* split (``fused=False`` or ``MINTCCL_ALLREDUCE=split``; the default from
  32 MiB per rank): a reduce-scatter launch followed by an allgather launch on
  the same chunks; each launch can use the whole wavefront budget, and the
  allgather's origins get compute units of their own.
"""
from __future__ import annotations

import os

import torch

from . import _lib
from ._ops import (check_buffer, comm_or_default, nbytes, reduce_dtype, ring_of,
                   same_everywhere)
from .common import VirtualComm


# From this size per rank on, two launches are faster than one pass (measured
# on MI355X, 8 ranks, f16: 104 / 110 us at 16 MiB, 199 / 192 at 32 MiB, 1510 /
# 1384 at 256 MiB; below, the second launch costs more than it gains: 12 / 18 us
# at 64 KiB).
SPLIT_FROM_BYTES = 32 << 20


def chunk_bytes(count: int, world: int) -> int:
    """Bytes of one chunk: ceil(count / world) rounded up to whole 16-byte vectors."""
    return (-(-count // world) + 15) // 16 * 16


def allreduce(buff: torch.Tensor, comm: VirtualComm | None = None,
              fused: bool | None = None) -> None:
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
    if fused is None:
        choice = os.getenv("MINTCCL_ALLREDUCE", "").lower()
        fused = choice != "split" if choice else count < SPLIT_FROM_BYTES
    ring = ring_of(comm)
    if fused:
        comm.launch(comm.make_op(_lib.OP_ALLREDUCE, dtype, count, ptrs, ptrs, ring))
        return
    row = chunk_bytes(count, comm.world_size)
    comm.launch(comm.make_op(_lib.OP_REDUCESCATTER, dtype, row, ptrs, ptrs, ring, row_stride=row,
                             total_bytes=count))
    comm.launch(comm.make_op(_lib.OP_ALLGATHER, _lib.BYTES, row, ptrs, ptrs, ring, row_stride=row,
                             total_bytes=count))


if __name__ == "__main__":      # the reference runs its self-test from here
    import sys

    from .selftest import main
    sys.exit(main("allreduce"))
