"""What the device does with the ring kernels' memory accesses when nothing
waits for anything: ``python -m mintccl_amd.yardsticks`` prints, one JSON line
each, the copy and read bandwidth of the library's own kernels on 1 GiB and
the time of the access mix of the headline launch (8 ranks x 256 MiB:
2,517,120 blocks of 1 KiB) spread over different numbers of wavefronts - per
wavefront and step a 960-byte own-row load from HBM, a 1 KiB load from and a
1 KiB store into staging that stays in L2, in every combination:

``mint_step_mix``       one step in flight per wavefront (load, wait, add,
                        store, next step), also with the own rows loaded
                        straight into LDS, and the mix of a copying position
                        (staging load, staging store, store to HBM);
                        and, for the headline's 4032 wavefronts, the whole mix
                        with 32 - 192 scalar instructions per step between
                        the loads and the store;
``mint_step_mix_deep``  the loads 1, 2 or 3 steps ahead of their use and the
                        stores never waited for: 2, 3 or 4 steps in flight per
                        wavefront, each line written by one compute unit and
                        read by another.

The ring kernels do exactly these accesses plus their flags, so these times
are what they are measured against.

``python -m mintccl_amd.yardsticks --counters [waves]`` launches, twice each
and for one wavefront count (default 4032, the headline launch's), the kernels
a counter run compares: the headline reduce-scatter itself, the mix at 1 - 4
steps in flight, its parts alone, the mix of a copying position, and the
read-only pass; meant to run under
``rocprofv3 --pmc``.  No counterpart in the reference.
"""
from __future__ import annotations

import json
import os
import sys

import torch

from . import primitive

BLOCKS = 5760 * 437           # 1 KiB blocks x hops of the headline launch
PARTS = (("own rows", 1), ("staging load", 2), ("staging store", 4), ("staging load + store", 6),
         ("own rows + staging store", 5), ("own rows + staging load", 3), ("all three", 7))


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


def steps_for(waves: int, ahead: int) -> int:
    """Steps per wavefront for the headline's block count, whole rounds of the
    unrolled loop."""
    iters = -(-BLOCKS // waves)
    return -(-iters // (ahead + 1)) * (ahead + 1)


def headline_launch(dev: torch.device):
    """The 8 x 256 MiB fp16 reduce-scatter at the library's tuned geometry:
    returns a function that enqueues one launch."""
    from .common import VirtualComm
    from .reducescatter import reducescatter
    world, n = 8, (256 << 20) // 2 // 8
    bufs = []
    for r in range(world):
        g = torch.Generator(device=dev).manual_seed(3000 + r)
        bufs.append(torch.randn(world, n, generator=g, device=dev, dtype=torch.float32)
                    .to(torch.float16))
    comm = VirtualComm(world_size=world, device=dev)
    return (lambda: comm.run(lambda r: reducescatter(bufs[r], comm))), comm


def counters(dev: torch.device, waves: int) -> int:
    launch, comm = headline_launch(dev)
    for _ in range(3):
        launch()
    comm.check()
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 256)
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    for _ in range(2):
        primitive.read_xor(src, sink)
    del src
    rows = torch.empty((BLOCKS + 8 * waves) * 960, dtype=torch.uint8, device=dev).random_(0, 256)
    staging = torch.zeros(waves * 5 * 1024, dtype=torch.uint8, device=dev)
    for _ in range(2):
        primitive.step_mix(rows, staging, waves, steps_for(waves, 0), 7)
        for ahead in (1, 2, 3):
            primitive.step_mix_deep(rows, staging, waves, steps_for(waves, ahead), 7, ahead)
        # the parts alone, three steps ahead: own rows; staging loads and stores
        primitive.step_mix_deep(rows, staging, waves, steps_for(waves, 3), 1, 3)
        primitive.step_mix_deep(rows, staging, waves, steps_for(waves, 3), 6, 3)
        primitive.step_mix_deep(rows, staging, waves, steps_for(waves, 3), 2, 3)
        primitive.step_mix_deep(rows, staging, waves, steps_for(waves, 3), 4, 3)
        # what a copying position does: the streaming store to HBM alone, and
        # with the staging load and store around it
        primitive.step_mix(rows, staging, waves, steps_for(waves, 0), 16)
        primitive.step_mix(rows, staging, waves, steps_for(waves, 0), 22)
    torch.cuda.synchronize()
    print(json.dumps({"counters": "launched", "wavefronts": waves}), flush=True)
    return 0


def main(argv: list[str]) -> int:
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    mask = os.getenv("MINTCCL_YARD_CU_MASK", "")
    if mask:
        # diagnostic: run on a stream restricted to some of the CUs (hex pattern
        # of 32 bits, repeated over the device: 00FF00FF leaves half of them)
        import ctypes
        hip = ctypes.CDLL("libamdhip64.so")
        words = (ctypes.c_uint32 * 8)(*([int(mask, 16)] * 8))
        handle = ctypes.c_void_p()
        if hip.hipExtStreamCreateWithCUMask(ctypes.byref(handle), 8, words) != 0:
            print("hipExtStreamCreateWithCUMask failed", file=sys.stderr)
            return 1
        torch.cuda.set_stream(torch.cuda.ExternalStream(handle.value))
        print(json.dumps({"cu_mask": mask}), flush=True)
    if argv and argv[0] == "--counters":
        return counters(dev, int(argv[1]) if len(argv) > 1 else 4032)
    deep_only = bool(argv) and argv[0] == "--deep"
    if deep_only:
        argv = argv[1:]
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 256)
    dst = torch.empty_like(src)
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    print(json.dumps({"yardstick": "copy 1 GiB", "gbps": round(
        2 * (1 << 30) / best_ms(lambda: primitive.copy128(src, dst)) / 1e6, 1)}), flush=True)
    print(json.dumps({"yardstick": "read 1 GiB", "gbps": round(
        (1 << 30) / best_ms(lambda: primitive.read_xor(src, sink)) / 1e6, 1)}), flush=True)
    del src, dst
    waves_list = [int(a) for a in argv] or [1440, 2016, 2880, 3600, 4032, 4320, 5040, 5760, 7200, 11520]
    rows = torch.empty((BLOCKS + 8 * max(waves_list)) * 960, dtype=torch.uint8,
                       device=dev).random_(0, 256)
    what = PARTS + (
        ("own rows into LDS", 9), ("own rows into LDS + staging store", 13),
        ("all three, own rows into LDS", 15),
        # what a copying position does: staging load, save to HBM, staging store
        ("HBM store", 16), ("staging load + HBM store", 18), ("staging store + HBM store", 20),
        ("staging load + staging store + HBM store", 22))
    for waves in waves_list:
        staging = torch.zeros(waves * 5 * 1024, dtype=torch.uint8, device=dev)
        if not deep_only and waves == 4032:
            # the whole mix with scalar instructions between the loads and the
            # store of every step: what a ring step's bookkeeping may cost
            iters = steps_for(waves, 0)
            line = {"yardstick": "step mix and scalar instructions", "wavefronts": waves, "steps": iters}
            for k in (0, 2, 4, 5, 6, 8, 12):
                line[f"all three + {16 * k} scalar ms"] = round(best_ms(
                    lambda b=7 + 256 * k: primitive.step_mix(rows, staging, waves, iters, b)), 4)
            print(json.dumps(line), flush=True)
        if not deep_only:
            iters = steps_for(waves, 0)
            line = {"yardstick": "step mix", "steps_in_flight": 1, "wavefronts": waves,
                    "steps": iters, "staging_mib": round(waves * 2048 / (1 << 20), 2)}
            for name, bits in what:
                line[name + " ms"] = round(best_ms(
                    lambda b=bits: primitive.step_mix(rows, staging, waves, iters, b)), 4)
            print(json.dumps(line), flush=True)
        for ahead in (1, 2, 3):
            iters = steps_for(waves, ahead)
            line = {"yardstick": "step mix", "steps_in_flight": ahead + 1, "wavefronts": waves,
                    "steps": iters, "staging_mib": round(waves * (ahead + 2) * 1024 / (1 << 20), 2)}
            for name, bits in PARTS:
                line[name + " ms"] = round(best_ms(
                    lambda b=bits, a=ahead, n=iters: primitive.step_mix_deep(
                        rows, staging, waves, n, b, a)), 4)
            # the same with every wavefront loading what it stored itself
            line["all three, own lines ms"] = round(best_ms(
                lambda a=ahead, n=iters: primitive.step_mix_deep(
                    rows, staging, waves, n, 7, a, partner=False)), 4)
            print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
