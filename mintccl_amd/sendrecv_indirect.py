"""Multi-hop LL128 send / recv with full-size staging
(``2_sendrecv_indirect.py``): every line of the message has a staging slot of
its own (``:147-149``), so no hop ever waits for a credit."""
from __future__ import annotations

from . import sendrecv_buffer as _buffered
from ._ops import comm_or_default
from .common import VirtualComm

send = _buffered.send
recv = _buffered.recv


def sync(comm: VirtualComm | None = None, route: list[int] | None = None) -> None:
    comm = comm_or_default(comm)
    st = _buffered._state(comm)
    if st["send"] is None or st["recv"] is None:
        return
    s, r = st["send"], st["recv"]
    st["send"] = st["recv"] = None
    _buffered._launch(comm, s, r, route, full_size_staging=True)


if __name__ == "__main__":      # the reference runs its self-test from here
    import sys

    from .selftest import main
    sys.exit(main("sendrecv_indirect"))
