"""Direct send / recv: the simple protocol (``1_sendrecv_direct.py``).

The sender only publishes its pointer (``1_sendrecv_direct.py:60-62``); the
receiver pulls with a persistent 16-byte-per-lane copy kernel (``:65-79``).
"""
from __future__ import annotations

import torch

from . import _lib
from ._ops import check_buffer, comm_or_default, nbytes
from .common import VirtualComm, num_blocks, num_warps


def send(buff: torch.Tensor, peer: int, comm: VirtualComm | None = None) -> None:
    comm = comm_or_default(comm)
    check_buffer(buff, comm)
    comm.send_ptr((buff.data_ptr(), nbytes(buff)), peer)


def recv(buff: torch.Tensor, peer: int, profile: bool = True,
         comm: VirtualComm | None = None) -> None:
    comm = comm_or_default(comm)
    check_buffer(buff, comm)
    sendbuff, sent = comm.recv_ptr(peer)
    count = nbytes(buff)
    if sent != count:
        raise ValueError(f"send posted {sent} bytes, recv expects {count}")
    with torch.cuda.device(comm.device):
        stream = torch.cuda.current_stream().cuda_stream
        # reference grid: NUM_BLOCKS blocks of NUM_WARPS warps; 0 lets the
        # library fill the device
        blocks = 0 if "MINTCCL_NUM_BLOCKS" not in __import__("os").environ else num_blocks()
        threads = min(1024, num_warps() * 32)
        _lib.check(_lib.lib().mint_copy_simple(sendbuff, buff.data_ptr(), count, blocks, threads,
                                               stream), "mint_copy_simple")
    if profile:                      # 1_sendrecv_direct.py:77-79
        torch.cuda.synchronize(comm.device)


if __name__ == "__main__":      # the reference runs its self-test from here
    import sys

    from .selftest import main
    sys.exit(main("sendrecv_direct"))
