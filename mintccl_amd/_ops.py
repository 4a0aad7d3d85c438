"""Shared plumbing of the operator modules: argument checks and the fused
launch once every participating rank has posted its buffer."""
from __future__ import annotations

import torch

from . import _lib
from .common import DTYPE_CODE, VirtualComm, get_comm
from .topology import find_ring, uniform_topology


def nbytes(t: torch.Tensor) -> int:
    return t.numel() * t.element_size()      # count = numel * itemsize (4_broadcast.py:80)


def check_buffer(t: torch.Tensor, comm: VirtualComm) -> None:
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TypeError("buffer must be a device tensor")
    if t.device != comm.device and t.device.index != comm.device.index:
        raise ValueError("buffer lives on another device than the communicator")
    if not t.is_contiguous():
        raise ValueError("buffer must be contiguous")


def ring_of(comm: VirtualComm) -> list[int]:
    """The ring of the communicator's topology (searched once per topology
    object: the search costs more than a small collective)."""
    topo = getattr(comm, "topology", None)
    cached = getattr(comm, "_ring_cache", None)
    if cached is not None and cached[0] is topo:
        return cached[1]
    ring = find_ring(topo or uniform_topology(comm.world_size))
    if len(ring) != comm.world_size + 1:
        raise RuntimeError("topology has no ring through every rank")
    comm._ring_cache = (topo, ring)
    return ring


def same_everywhere(posted: dict, field: str, what: str):
    vals = {info[field] for info in posted.values()}
    if len(vals) != 1:
        raise ValueError(f"ranks disagree on {what}: {sorted(map(str, vals))}")
    return vals.pop()


def reduce_dtype(t: torch.Tensor) -> int:
    if t.dtype not in DTYPE_CODE:
        raise TypeError("reductions take float16, bfloat16 or float32 tensors")
    return DTYPE_CODE[t.dtype]


def comm_or_default(comm: VirtualComm | None) -> VirtualComm:
    return comm if comm is not None else get_comm()
