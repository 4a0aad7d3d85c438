#!/usr/bin/env python3
"""Headline benchmark: 8-virtual-rank LL128 ring reduce-scatter, fp16, 256 MiB
per rank, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one fused launch that runs all 8 ranks' kernels over inputs that
are already resident in HBM.  Prints ONE JSON line:

  value     bytes that have to cross HBM per step - every rank reads its whole
            buffer once (N S) and the N reduced chunks are written (S):
            (N + 1) S = 2.416 GB - over the time of a step, GB/s.  A step is
            one launch, timed by events on the launch stream; between the
            launches the inputs are put back (the collective works in place),
            so every timed launch reduces the stated normal(0, 1) values, and
            the first and the last launch are verified.
  roofline  the same bytes over the kernel's own duration (events on the
            launch stream) against the 8 TB/s HBM peak: a fraction <= 1.
            `traffic` = HBM bytes per launch measured with rocprofv3 counters,
            read from the committed summary of exactly this geometry
            (profiles/*_pmc.txt), null for any other geometry.
  algorithmic_gbps  the ring's payload, (3 N + 1) S = 6.711 GB per step (per
            chunk: N own-row reads, N staging writes, N staging reads, 1
            result write), over the kernel's duration.  Two thirds of it are
            staging bytes that stay in the L2 of the XCD that hosts the
            channel, so this is NOT an HBM rate.
  l2        bytes the L2 serves per launch (requests counted by rocprofv3,
            128 B per read, 64 B per write, same profile) over the kernel's
            duration, against 128 channels x 128 B x 2.4 GHz.
  step_mix  the same number of wavefronts doing the loads and stores of the
            same number of ring steps with no flags and no waiting
            (mint_step_mix): what the device needs for this mix of accesses.
  copy_* / read_*  measured HBM copy and read bandwidth of the library's own
            16 B / lane kernels on 1 GiB.
  cpu_baseline  the PyTorch-CPU walk of the same collective through the same
            wire format (oracle/torch_ring.py), timed on this host;
            cpu_baseline_c is the C / OpenMP restatement of the walk.
"""
from __future__ import annotations

import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

WORLD = 8
PER_RANK_BYTES = 256 << 20
HBM_PEAK_GBPS = 8000.0
L2_PEAK_GBPS = 128 * 128 * 2.4          # 128 channels x 128 B per clock x 2.4 GHz

# launch geometry used for the headline (the library's tuned default for this
# collective): 3 slots of 448 KiB per rank, so that all staging of an XCD's
# channels stays in its 4 MiB L2, 56 wave-channels per (chunk, hop) in thread
# blocks of two, every hop of a channel on one XCD
BUFF_BYTES = int(os.getenv("MINTCCL_BENCH_BUFF", 3 * 448 * 1024))
NSLOTS = int(os.getenv("MINTCCL_BENCH_NSLOTS", 3))
WAVES_PER_RANK = int(os.getenv("MINTCCL_BENCH_WAVES", 448))
THREADS = int(os.getenv("MINTCCL_BENCH_THREADS", 128))
PLACEMENT = int(os.getenv("MINTCCL_BENCH_PLACEMENT", 1))      # 0 spread, 1 local
CACHE_POLICY = int(os.getenv("MINTCCL_BENCH_CACHE", 2))       # 0 agent, 1 system, 2 XCD-local
ROW_FETCH = int(os.getenv("MINTCCL_BENCH_FETCH", 0))          # 0 in registers, 1 through LDS
# Diagnostic: run on a stream restricted to some of the CUs (hex pattern of 32
# bits, repeated over the device's CUs; 00FF00FF leaves half of the CUs of
# every XCD) to tell a per-CU limit from a device-wide one.  A grid that is no
# longer co-resident still finishes: a channel's positions are dispatched together.
CU_MASK = os.getenv("MINTCCL_BENCH_CU_MASK", "")


def geometry_key() -> str:
    return (f"world={WORLD} per_rank={PER_RANK_BYTES} buff={BUFF_BYTES} nslots={NSLOTS} "
            f"waves={WAVES_PER_RANK} threads={THREADS} placement={PLACEMENT} cache={CACHE_POLICY} "
            f"fetch={ROW_FETCH}")


def profiled(field: str):
    """`field` of the committed rocprofv3 summary taken at exactly this launch
    geometry: (value, file name), or (None, None)."""
    pdir = os.path.join(ROOT, "profiles")
    if not os.path.isdir(pdir):
        return None, None
    for name in sorted(os.listdir(pdir)):
        if not name.endswith(".txt"):
            continue
        text = open(os.path.join(pdir, name)).read()
        if f"bench geometry: {geometry_key()}" not in text:
            continue
        m = re.search(rf"^{field}\s*=\s*([0-9.eE+]+)", text, flags=re.M)
        if m:
            return float(m.group(1)), name
    return None, None


def cpu_baselines(seconds_budget: float = 25.0) -> dict:
    """The CPU restatements of the same collective, timed on this host: the
    PyTorch-CPU walk on the full workload and the C / OpenMP walk on an eighth
    of it."""
    import numpy as np
    import torch
    from oracle import cref, torch_ring
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    n = PER_RANK_BYTES // 2 // WORLD
    g = torch.Generator().manual_seed(3000)
    bufs = [torch.randn(WORLD, n, generator=g).to(torch.float16) for _ in range(WORLD)]
    t_end = time.perf_counter() + seconds_budget
    torch_ring.reducescatter_wire(bufs, "f16")                 # warm-up
    times = []
    while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 5):
        t0 = time.perf_counter_ns()
        torch_ring.reducescatter_wire(bufs, "f16")
        times.append((time.perf_counter_ns() - t0) / 1e9)
    med = sorted(times)[len(times) // 2]
    hbm_bytes = (WORLD + 1) * PER_RANK_BYTES
    out = {"cpu_baseline": {
        "value": round(hbm_bytes / med / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(),
        "kind": "port", "seconds_per_step": round(med, 3),
        "algorithmic_gbps": round((3 * WORLD + 1) * PER_RANK_BYTES / med / 1e9, 3),
        "sample": f"PyTorch-CPU walk of the same reduce-scatter through the LL128 wire format "
                  f"(oracle/torch_ring.py), the full workload: 8 ranks x {PER_RANK_BYTES >> 20} MiB "
                  f"fp16, 1 warm-up + median of {len(times)} runs; value = (N + 1) S bytes per second"}}
    del bufs
    threads = min(cores, int(os.getenv("OMP_NUM_THREADS", cores)))
    per_rank = 32 << 20
    rng = np.random.default_rng(3000)
    small = [rng.standard_normal(per_rank // 2, dtype=np.float32).astype(np.float16).view(np.uint8)
             for _ in range(WORLD)]
    cref.reducescatter_wire([b.copy() for b in small], "f16", threads=threads)
    times = []
    for _ in range(3):
        work = [b.copy() for b in small]
        t0 = time.perf_counter_ns()
        bad = cref.reducescatter_wire(work, "f16", threads=threads)
        times.append((time.perf_counter_ns() - t0) / 1e9)
        assert bad == 0
    med = sorted(times)[1]
    out["cpu_baseline_c"] = {
        "value": round((WORLD + 1) * per_rank / med / 1e9, 3), "unit": "GB/s", "cores": threads,
        "kind": "port", "algorithmic_gbps": round((3 * WORLD + 1) * per_rank / med / 1e9, 3),
        "sample": f"the same walk in C / OpenMP (oracle/ll128_ref.c), 8 ranks x {per_rank >> 20} MiB "
                  f"fp16 (an eighth of the workload), median of 3 runs"}
    return out


def best_ms(fn, reps: int = 5) -> float:
    import torch
    for _ in range(2):
        fn()
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(); fn(); e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1))
    return best


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--also-64mib", action="store_true",
                    help="also time the same collective at 64 MiB per rank (the baseline's "
                         "configuration 4 reading of the headline); off by default so that every "
                         "launch of the ring kernel in a profile of this command is a headline launch")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.getenv("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU (the 8 ring ranks are disjoint HBM regions "
              "of one MI355X); --gpus must be 1", file=sys.stderr)
        return 2

    import torch
    from mintccl_amd import _lib, primitive
    from mintccl_amd.common import VirtualComm
    from mintccl_amd.reducescatter import reducescatter

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if CU_MASK:
        import ctypes
        hip = ctypes.CDLL("libamdhip64.so")
        words = (ctypes.c_uint32 * 8)(*([int(CU_MASK, 16)] * 8))
        handle = ctypes.c_void_p()
        if hip.hipExtStreamCreateWithCUMask(ctypes.byref(handle), 8, words) != 0:
            print("bench.py: hipExtStreamCreateWithCUMask failed", file=sys.stderr)
            return 1
        torch.cuda.set_stream(torch.cuda.ExternalStream(handle.value))

    # yardsticks: the library's own copy and read-only kernels on 1 GiB
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 256)
    dst = torch.empty_like(src)
    copy_gbps = 2 * (1 << 30) / best_ms(lambda: primitive.copy128(src, dst)) / 1e6
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    read_gbps = (1 << 30) / best_ms(lambda: primitive.read_xor(src, sink)) / 1e6
    del src, dst

    # synthetic input: normal(0,1) drawn per rank (seed 3000 + rank), fp16
    n = PER_RANK_BYTES // 2 // WORLD
    bufs = []
    for r in range(WORLD):
        g = torch.Generator(device=dev).manual_seed(3000 + r)
        bufs.append(torch.randn(WORLD, n, generator=g, device=dev, dtype=torch.float32)
                    .to(torch.float16))
    comm = VirtualComm(world_size=WORLD, device=dev, buff_size_=BUFF_BYTES, nslots=NSLOTS,
                       waves_per_rank=WAVES_PER_RANK, threads_per_block=THREADS,
                       placement=PLACEMENT, cache_policy=CACHE_POLICY, row_fetch=ROW_FETCH)

    def step():
        comm.run(lambda r: reducescatter(bufs[r], comm))

    # the first launch is checked: every owner row against the device adder
    # folded in ring order (own + received, starting from the owner's value)
    # on untouched copies of the inputs, every other row unchanged
    orig = [b.clone() for b in bufs]
    step()
    comm.check()
    verified = True
    for c in range(WORLD):
        acc = orig[c][c].clone()
        for k in range(1, WORLD):
            acc = primitive.Sum(orig[(c + k) % WORLD][c].contiguous(), acc)
        verified &= torch.equal(bufs[c][c].view(torch.int16), acc.view(torch.int16))
        for r in range(WORLD):
            if r != c:
                verified &= torch.equal(bufs[r][c].view(torch.int16), orig[r][c].view(torch.int16))
    del acc
    if not verified:
        print("bench.py: the reduce-scatter result is wrong", file=sys.stderr)
        return 1

    def restore():
        # the collective works in place: every launch gets the stated inputs
        # (normal(0, 1) values, not the sums the launch before left behind)
        for b, o in zip(bufs, orig):
            b.copy_(o)

    def verify() -> bool:
        ok = True
        for c in range(WORLD):
            acc = orig[c][c].clone()
            for k in range(1, WORLD):
                acc = primitive.Sum(orig[(c + k) % WORLD][c].contiguous(), acc)
            ok &= torch.equal(bufs[c][c].view(torch.int16), acc.view(torch.int16))
            for r in range(WORLD):
                if r != c:
                    ok &= torch.equal(bufs[r][c].view(torch.int16), orig[r][c].view(torch.int16))
        return bool(ok)

    for _ in range(args.warmup):
        restore()
        step()
    comm.check()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        restore()                     # outside the timed region: 2 GiB of copies per step
        starts[i].record()
        step()
        stops[i].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    comm.check()
    # the last timed launch is checked like the first
    verified = verified and verify()
    if not verified:
        print("bench.py: the last timed reduce-scatter is wrong", file=sys.stderr)
        return 1
    kernel_ms = sum(s.elapsed_time(e) for s, e in zip(starts, stops)) / args.steps

    small_ms = None
    if args.also_64mib:
        # the other reading of the baseline's headline (its config 4: 32 Mi
        # elements = 64 MiB per rank), same launch geometry, labelled as such
        small = [b[:, : n // 4] .contiguous() for b in bufs]

        def small_step():
            comm.run(lambda r: reducescatter(small[r], comm))

        for _ in range(args.warmup):
            small_step()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(args.steps):
            small_step()
        e1.record()
        torch.cuda.synchronize()
        comm.check()
        small_ms = e0.elapsed_time(e1) / args.steps
        del small

    # the loads and stores of the same launch with nothing waiting for anything
    wave_channels = WAVES_PER_RANK * (WORLD + 1)          # one per (chunk, position, channel)
    blocks_per_row = -(-(PER_RANK_BYTES // WORLD) // 960)
    iters = -(-blocks_per_row // (WAVES_PER_RANK // WORLD))
    rows = torch.empty(wave_channels * iters * 960, dtype=torch.uint8, device=dev).random_(0, 256)
    scratch = torch.zeros(wave_channels * 2048, dtype=torch.uint8, device=dev)
    mix_ms = best_ms(lambda: primitive.step_mix(rows, scratch, wave_channels, iters, 7))
    del rows, scratch

    hbm_bytes = (WORLD + 1) * PER_RANK_BYTES                # what has to cross HBM
    payload = (3 * WORLD + 1) * PER_RANK_BYTES              # what the ring moves
    # A step is the launch (events around it on the launch stream); the copies
    # that put the inputs back between the launches are not part of it.  The
    # wall time of the loop, copies included, is reported beside it.
    ms_per_step = kernel_ms
    wall_ms_per_step = wall * 1e3 / args.steps
    value = hbm_bytes / (ms_per_step / 1e3) / 1e9
    achieved = hbm_bytes / (kernel_ms / 1e3) / 1e9
    algorithmic = payload / (kernel_ms / 1e3) / 1e9
    algbw = PER_RANK_BYTES / (kernel_ms / 1e3) / 1e9
    traffic, traffic_file = profiled("traffic_bytes_per_launch")
    l2_bytes, l2_file = profiled("l2_bytes_per_launch")
    l2_req, _ = profiled("l2_requests_per_launch")
    out = {
        "metric": "achieved HBM GB/s and % of roofline, 8-rank LL128 reducescatter 256MiB fp16",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "value_definition": "(N + 1) S = 2,415,919,104 bytes that must cross HBM per step (N S of "
                            "input read, S of result written) / time per step (events around "
                            "each launch; every launch reduces freshly restored normal(0,1) "
                            "inputs, first and last launch verified)",
        "wall_ms_per_step_with_input_restore": round(wall_ms_per_step, 4),
        "verified": verified,
        "config": {"workload": "ring reducescatter, LL128 (64-byte-sector tags), 8 virtual ranks "
                               "x 256 MiB fp16 on one MI355X, in place",
                   "world": WORLD, "per_rank_bytes": PER_RANK_BYTES, "staging_per_rank": BUFF_BYTES,
                   "nslots": NSLOTS, "waves_per_rank": WAVES_PER_RANK, "threads": THREADS,
                   "placement": ["spread", "local"][PLACEMENT],
                   "staging_cache_policy": ["agent", "system", "xcd-local"][CACHE_POLICY],
                   "own_rows": ["registers", "lds"][ROW_FETCH], "cu_mask": CU_MASK or None,
                   "library_build_flags": _lib.build_flags(),
                   "grid_blocks": comm.last_grid, "hbm_bytes_per_step": hbm_bytes,
                   "payload_bytes_per_step": payload},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": traffic, "traffic_profile": traffic_file},
        "kernel_ms": round(kernel_ms, 4),
        # the ring's payload: two thirds of it never leave the per-XCD L2
        "algorithmic_gbps": round(algorithmic, 1),
        "copy_bw_gbps": round(copy_gbps, 1),
        "algorithmic_frac_of_copy_bw": round(algorithmic / copy_gbps, 4),
        "hbm_frac_of_copy_bw": round(achieved / copy_gbps, 4),
        "read_bw_gbps": round(read_gbps, 1),
        "hbm_frac_of_read_bw": round(achieved / read_gbps, 4),
        "l2": None if l2_bytes is None else {
            "bytes_per_launch": l2_bytes, "requests_per_launch": l2_req,
            "achieved": round(l2_bytes / (kernel_ms / 1e3) / 1e9, 1), "peak": round(L2_PEAK_GBPS, 1),
            "unit": "GB/s", "frac": round(l2_bytes / (kernel_ms / 1e3) / 1e9 / L2_PEAK_GBPS, 4),
            "profile": l2_file},
        "step_mix": {"ms": round(mix_ms, 4), "wavefronts": wave_channels, "steps_per_wavefront": iters,
                     "kernel_over_mix": round(kernel_ms / mix_ms, 4),
                     "what": "own-row load + staging load + staging store per step, no flags, "
                             "no waiting (mint_step_mix)"},
        "algbw_gbps": round(algbw, 1), "busbw_gbps": round(algbw * (WORLD - 1) / WORLD, 1),
        "flag_bytes_frac_of_staging": round(8 / 128, 4),
    }
    if small_ms is not None:
        out["at_64mib_per_rank"] = {
            "workload": "same collective, 64 MiB fp16 per rank (32 Mi elements)",
            "ms_per_step": round(small_ms, 4),
            "hbm_gbps": round((WORLD + 1) * (PER_RANK_BYTES // 4) / (small_ms / 1e3) / 1e9, 1)}
    if not args.no_cpu_baseline:
        out.update(cpu_baselines())
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
