"""Where the wave-channels of a collective spend a step: ``python -m
mintccl_amd.waits [reducescatter allgather ...]`` launches the named
collectives (default: the 8 x 256 MiB reduce-scatter and the 8 x 128 MiB
allgather) at the tuned geometry and prints, per ring position, the averages a
wave-channel collects in a library built with ``-DMINT_RING_STATS``:

    python -c "from mintccl_amd import _lib; _lib.build(defines=('-DMINT_RING_STATS',), so_path='/tmp/libstats.so')"
    MINTCCL_LIBRARY=/tmp/libstats.so python -m mintccl_amd.waits

The product library does not collect them (it refuses a stats address): the
accounting costs scalar registers and a few per cent of time, more on kernels
shorter than a millisecond.  Per step and wave-channel, in nanoseconds:
``credit`` waiting for the next rank to free the slot, ``poll`` waiting for
the tags of the step (``re-polls`` = repeated polls per step), ``own rows``
waiting for rows fetched ahead (LL128 copying walks; for the walk with own
rows through LDS, the wait for the fetcher), ``issue`` handing the step's
loads and stores to the memory pipeline (LL128 copying walks), ``total`` the
whole step.  No counterpart in the reference.
"""
from __future__ import annotations

import json
import sys

import torch

from . import _lib, common

WORLD = 8


def account(comm: common.VirtualComm, make) -> dict:
    """Time the launch ``make()`` describes without accounting, then once with."""
    dev = comm.device
    d = make()
    comm.launch(d)
    comm.check()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(4):
        comm.launch(d)
    e1.record()
    torch.cuda.synchronize()
    plain = e0.elapsed_time(e1) / 4
    comm.stats = torch.zeros(9 * 8, dtype=torch.int64, device=dev)
    try:
        d = make()
        e0.record()
        comm.launch(d)
        e1.record()
        torch.cuda.synchronize()
        comm.check()
        rows = comm.stats.cpu().view(9, 8).tolist()
    finally:
        comm.stats = None
    out = {"ms": round(plain, 4), "ms_with_accounting": round(e0.elapsed_time(e1), 4),
           "grid": comm.last_grid, "positions": []}
    for h, (groups, repolls, t_credit, t_poll, t_all, waves, t_rows, t_issue) in enumerate(rows):
        if not waves:
            continue
        g = max(groups, 1)
        out["positions"].append({
            "position": h, "wave_channels": waves, "steps": round(groups / waves),
            "re_polls": round(repolls / g, 2), "credit_ns": round(10 * t_credit / g),
            "poll_ns": round(10 * t_poll / g), "own_rows_ns": round(10 * t_rows / g),
            "issue_ns": round(10 * t_issue / g), "total_ns": round(10 * t_all / g)})
    return out


def main(argv: list[str]) -> int:
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    names = argv or ["reducescatter", "allgather"]
    ring = list(range(WORLD)) + [0]
    shard = 128 << 20
    bufs = [torch.zeros(WORLD, shard // 2, device=dev, dtype=torch.float16) for _ in range(WORLD)]
    ptrs = {r: bufs[r].data_ptr() for r in range(WORLD)}
    rest = {r: p for r, p in ptrs.items() if r}
    comm = common.VirtualComm(world_size=WORLD)
    cases = {
        "reducescatter": ("reducescatter, 8 x 256 MiB f16", lambda: comm.make_op(
            _lib.OP_REDUCESCATTER, _lib.F16, shard // 4, ptrs, ptrs, ring, row_stride=shard // 4)),
        "allgather": ("allgather, 8 x 128 MiB", lambda: comm.make_op(
            _lib.OP_ALLGATHER, _lib.BYTES, shard, ptrs, ptrs, ring, row_stride=shard)),
        "allreduce": ("allreduce in one pass, 256 MiB f16", lambda: comm.make_op(
            _lib.OP_ALLREDUCE, _lib.F16, 256 << 20, ptrs, ptrs, ring)),
        "broadcast": ("broadcast, 64 MiB", lambda: comm.make_op(
            _lib.OP_BROADCAST, _lib.BYTES, 64 << 20, {0: ptrs[0]}, rest, ring, root=0)),
        "reduce": ("reduce, 64 MiB f16", lambda: comm.make_op(
            _lib.OP_REDUCE, _lib.F16, 64 << 20, ptrs, {0: ptrs[0]}, ring, root=0)),
        "sendrecv": ("sendrecv, 256 MiB", lambda: comm.make_op(
            _lib.OP_SENDRECV, _lib.BYTES, 256 << 20, {0: ptrs[0]}, {1: ptrs[1]}, [0, 1],
            route_len=2)),
    }
    for name in names:
        if name not in cases:
            print(f"unknown collective {name!r}: one of {', '.join(cases)}", file=sys.stderr)
            return 2
    for name in names:
        title, make = cases[name]
        try:
            got = account(comm, make)
        except _lib.MintError as e:
            print(f"{title}: {e} (is MINTCCL_LIBRARY a -DMINT_RING_STATS build?)", file=sys.stderr)
            return 1
        print(json.dumps({"collective": title, "protocol": "ll128", **got}), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
