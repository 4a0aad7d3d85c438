"""Multi-hop LL128 send / recv with full-size staging
(``2_sendrecv_indirect.py``): every line of the message has a staging slot of
its own (``:147-149``), so no hop ever waits for a credit."""
from __future__ import annotations

import torch

from . import _lib, sendrecv_buffer as _buffered
from ._ops import comm_or_default
from .common import VirtualComm
from .protocol import packed_bytes

send = _buffered.send
recv = _buffered.recv


def sync(comm: VirtualComm | None = None, route: list[int] | None = None) -> None:
    comm = comm_or_default(comm)
    st = _buffered._state(comm)
    if st["send"] is None or st["recv"] is None:
        return
    s, r = st["send"], st["recv"]
    st["send"] = st["recv"] = None
    slot = comm.slot_bytes
    nslots = max(1, -(-packed_bytes(s["count"]) // slot))
    per_rank = nslots * slot + max(4096, slot // 4)
    # zeroed like the reference's (2_sendrecv_indirect.py:147); kept alive until
    # the next transfer replaces it, since the launch is asynchronous
    hops = torch.zeros(comm.world_size * per_rank, dtype=torch.uint8, device=comm.device)
    comm._indirect_staging = hops
    staging = {k: hops.data_ptr() + k * per_rank for k in range(comm.world_size)}
    _buffered._launch(comm, s, r, route, staging, (slot, nslots))
