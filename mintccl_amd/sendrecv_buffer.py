"""Multi-hop LL128 send / recv through fixed circular staging
(``3_sendrecv_buffer.py``).

``send`` and ``recv`` only record their arguments (``:78-92``); ``sync``,
called by every rank (``:98``), matches them, picks the route and enqueues one
launch in which every rank on the route runs its hop.
"""
from __future__ import annotations

import torch

from . import _lib
from ._ops import check_buffer, comm_or_default, nbytes
from .common import VirtualComm
from .protocol import packed_bytes
from .topology import find_route, uniform_topology

_KEY = "sendrecv_buffer"


def _state(comm: VirtualComm) -> dict:
    return comm.__dict__.setdefault("_" + _KEY, {"send": None, "recv": None})


def send(buff: torch.Tensor, peer: int, comm: VirtualComm | None = None) -> None:
    comm = comm_or_default(comm)
    check_buffer(buff, comm)
    _state(comm)["send"] = {"rank": comm.Get_rank(), "data_ptr": buff.data_ptr(),
                            "count": nbytes(buff), "dst": peer, "keep": buff}


def recv(buff: torch.Tensor, peer: int, comm: VirtualComm | None = None) -> None:
    comm = comm_or_default(comm)
    check_buffer(buff, comm)
    _state(comm)["recv"] = {"rank": comm.Get_rank(), "data_ptr": buff.data_ptr(),
                            "count": nbytes(buff), "src": peer, "keep": buff}


def _launch(comm: VirtualComm, s: dict, r: dict, route: list[int] | None,
            full_size_staging: bool = False) -> None:
    # 3_sendrecv_buffer.py:111-113
    if s["dst"] != r["rank"] or r["src"] != s["rank"]:
        raise ValueError("send and recv do not name each other")
    if s["count"] != r["count"]:
        raise ValueError("send and recv sizes differ")
    if route is None:
        topo = getattr(comm, "topology", None) or uniform_topology(comm.world_size)
        route = find_route(s["rank"], r["rank"], topo)
    if not route or route[0] != s["rank"] or route[-1] != r["rank"]:
        raise ValueError(f"no route {s['rank']} -> {r['rank']}")
    comm.last_route = list(route)
    d = comm.make_op(_lib.OP_SENDRECV, _lib.BYTES, s["count"], {s["rank"]: s["data_ptr"]},
                     {r["rank"]: r["data_ptr"]}, route, route_len=len(route))
    if full_size_staging:
        # every line of the message gets a slot of its own, so no hop ever
        # waits for a credit (2_sendrecv_indirect.py:147-149); zeroed like the
        # reference's, and kept alive until the next transfer replaces it,
        # since the launch is asynchronous
        slot = d.slot_bytes
        d.nslots = max(1, -(-packed_bytes(s["count"]) // slot))
        per_rank = d.nslots * slot + max(4096, slot // 4) + _lib.TICKET_BYTES
        hops = torch.zeros(comm.world_size * per_rank, dtype=torch.uint8, device=comm.device)
        comm._indirect_staging = hops
        for k in range(comm.world_size):
            d.staging[k] = hops.data_ptr() + k * per_rank
        d.staging_bytes = per_rank
        d.credit_offset = 0                      # right after this staging's own slots
    comm.launch(d)


def sync(comm: VirtualComm | None = None, route: list[int] | None = None) -> None:
    """Every rank calls this; the first call that finds a matched send / recv
    pair launches, the others find nothing left to do."""
    comm = comm_or_default(comm)
    st = _state(comm)
    if st["send"] is None or st["recv"] is None:
        return
    s, r = st["send"], st["recv"]
    st["send"] = st["recv"] = None
    _launch(comm, s, r, route)


if __name__ == "__main__":      # the reference runs its self-test from here
    import sys

    from .selftest import main
    sys.exit(main("sendrecv_buffer"))
