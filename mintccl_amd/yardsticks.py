"""What the device does with the ring kernels' memory accesses when nothing
waits for anything: ``python -m mintccl_amd.yardsticks`` prints, one JSON line
each, the copy and read bandwidth of the library's own kernels on 1 GiB and
the time of ``mint_step_mix`` - per wavefront and step a 960-byte own-row load
from HBM, a 1 KiB load from and a 1 KiB store into a private staging slot, in
every combination, also with the own rows loaded straight into LDS, and the
mix of a copying position (staging load, staging store, store to HBM) - for the block count of the headline launch (8 ranks x
256 MiB: 2,517,120 blocks of 1 KiB) spread over different numbers of
wavefronts.  The ring kernels do exactly these accesses plus their flags, so
these times are what they are measured against.  No counterpart in the
reference.
"""
from __future__ import annotations

import json
import sys

import torch

from . import primitive

BLOCKS = 5760 * 437           # 1 KiB blocks x hops of the headline launch


def best_ms(fn, reps: int = 5) -> float:
    for _ in range(2):
        fn()
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1))
    return best


def main(argv: list[str]) -> int:
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 256)
    dst = torch.empty_like(src)
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    print(json.dumps({"yardstick": "copy 1 GiB", "gbps": round(
        2 * (1 << 30) / best_ms(lambda: primitive.copy128(src, dst)) / 1e6, 1)}), flush=True)
    print(json.dumps({"yardstick": "read 1 GiB", "gbps": round(
        (1 << 30) / best_ms(lambda: primitive.read_xor(src, sink)) / 1e6, 1)}), flush=True)
    del dst
    waves_list = [int(a) for a in argv] or [1440, 2880, 3600, 4320, 5040, 5760, 7200, 11520]
    rows = torch.empty((BLOCKS + max(waves_list)) * 960, dtype=torch.uint8, device=dev).random_(0, 256)
    what = (("own rows", 1), ("staging load", 2), ("staging store", 4), ("staging load + store", 6),
            ("own rows + staging store", 5), ("own rows + staging load", 3), ("all three", 7),
            ("own rows into LDS", 9), ("own rows into LDS + staging store", 13),
            ("all three, own rows into LDS", 15),
            # what a copying position does: staging load, save to HBM, staging store
            ("HBM store", 16), ("staging load + HBM store", 18), ("staging store + HBM store", 20),
            ("staging load + staging store + HBM store", 22))
    for waves in waves_list:
        iters = -(-BLOCKS // waves)
        staging = torch.zeros(waves * 2048, dtype=torch.uint8, device=dev)
        line = {"yardstick": "step mix", "wavefronts": waves, "steps": iters,
                "staging_mib": round(waves * 2048 / (1 << 20), 2)}
        for name, bits in what:
            line[name + " ms"] = round(best_ms(
                lambda b=bits: primitive.step_mix(rows, staging, waves, iters, b)), 4)
        print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
