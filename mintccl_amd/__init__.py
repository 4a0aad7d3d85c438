"""mintccl_amd - the collective data path of MinTCCL for one MI355X (gfx950).

Operator surface (same names and argument order as the reference scripts):

    sendrecv_direct.send / recv                 1_sendrecv_direct.py
    sendrecv_indirect.send / recv / sync        2_sendrecv_indirect.py
    sendrecv_buffer.send / recv / sync          3_sendrecv_buffer.py
    broadcast.broadcast(buff, root)             4_broadcast.py
    reduce.reduce(buff, root)                   5_reduce.py
    allgather.allgather(buff)                   6_allgather.py
    reducescatter.reducescatter(buff)           7_reducescatter.py
    allreduce.allreduce(buff)                   8_allreduce.py (planned there, README.md:23)

plus ``common`` (knobs, ``VirtualComm``), ``primitive``, ``protocol`` and
``topology``.  All compute runs in ``libmintccl.so`` (hand-written HIP); the
package raises if that library has not been built.
"""
from . import _lib  # noqa: F401
from .common import VirtualComm, RingTimeout, get_comm, set_comm  # noqa: F401

__all__ = ["VirtualComm", "RingTimeout", "get_comm", "set_comm"]
