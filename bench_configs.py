#!/usr/bin/env python3
"""Throughput of the other benchmark configurations on one MI355X (bench.py
covers the headline).  One JSON line per measurement; every case is also
checked for correctness (bit-exact copies; reductions against the device
adder folded in ring order).

    python bench_configs.py [--quick]

  config 1  LL128 line codec alone: pack + unpack of 1 MiB (524,288 fp16) and of 256 MiB,
            the reference's 8-lane pair layout and the 64-lane block layout
  config 2  sendrecv 256 MiB fp16, rank 0 -> rank 1: LL128, Simple, direct copy
  config 3  ring broadcast 64 MiB, 8 ranks, 8 x 512 KiB slots
  config 4  ring reduce and reducescatter, 32 Mi elements per rank, f16 / bf16 / f32
  config 5  ring allgather sweep, shard 512 B .. 128 MiB, LL128 vs Simple
  next      ring allreduce (the reference's planned 8_allreduce), 64 and 256 MiB fp16;
            alltoall (its planned 9_alltoall), 64 and 256 MiB fp16 per rank

    --staging reference|tuned   only the geometry the configuration names, or
                                only the library's tuned default (a profile of one
                                such run has one launch shape per kernel name)

Algorithmic bytes (`alg_gbps`: what the ring moves, staging included): copy 2S;
sendrecv over h hops (2 + 2h) S; broadcast / allgather (3N - 2) S; reduce /
reducescatter (3N + 1) S; alltoall 4 N S.  `hbm_gbps` counts only what has to
cross HBM - inputs read once, results written once: sendrecv 2S, broadcast N S,
allgather N S (S = N shards), reduce / reducescatter (N + 1) S, allreduce
2 N S, alltoall 2 N S.
"""
from __future__ import annotations

import argparse
import json
import os
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import torch  # noqa: E402

from mintccl_amd import _lib, primitive, protocol, sendrecv_buffer, sendrecv_direct  # noqa: E402
from mintccl_amd.allgather import allgather  # noqa: E402
from mintccl_amd.broadcast import broadcast  # noqa: E402
from mintccl_amd.common import VirtualComm  # noqa: E402
from mintccl_amd.reduce import reduce  # noqa: E402
from mintccl_amd.reducescatter import reducescatter  # noqa: E402

DEV = torch.device("cuda:0")
TDT = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}


def time_ms(fn, reps: int) -> float:
    """Average device time of `reps` back-to-back launches (the host side of a
    launch hides behind the previous kernel)."""
    fn()
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(2):      # twice, keep the better: a one-off host stall does not count
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        fn()
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1) / reps)
    return best


STAGING = ("reference", "tuned")      # set from --staging


def geometries(reference_label: str, slots):
    """(label, slots) pairs to run: the geometry the configuration names and /
    or the library's tuned default."""
    out = []
    if "reference" in STAGING:
        out.append((reference_label, slots))
    if "tuned" in STAGING:
        out.append(("tuned", None))
    return out


def emit(**kw) -> None:
    if "hbm_bytes" in kw:
        t = kw["ms"] if "ms" in kw else kw["us"] / 1e3
        kw["hbm_gbps"] = round(kw.pop("hbm_bytes") / t / 1e6, 1)
    print(json.dumps(kw), flush=True)


def comm_for(world: int, proto: int, slots=None, **kw) -> VirtualComm:
    """slots = (nslots, slot_bytes) for the geometry the configuration names;
    None = the library's tuned default."""
    if slots is not None:
        kw.update(buff_size_=slots[0] * slots[1], nslots=slots[0])
    return VirtualComm(world_size=world, device=DEV, protocol=proto, **kw)


def config1(reps: int) -> None:
    """The codec on its own: raw -> lines -> raw (mint_ll128_pack / _unpack),
    flag = line number from 1 as in the reference.  Bytes that cross HBM:
    raw read + lines written, lines read + raw written."""
    for n in (524288, 134217728):
        g = torch.Generator(device=DEV).manual_seed(0)
        raw = torch.empty(n, device=DEV, dtype=torch.float16).uniform_(-1, 1, generator=g)
        back = torch.empty_like(raw)
        bad = torch.zeros(1, dtype=torch.int64, device=DEV)
        for name, layout in (("pair (8 lanes, the reference's)", protocol.LAYOUT_PAIR),
                             ("wave64 (1 KiB blocks)", protocol.LAYOUT_WAVE64)):
            msg = torch.empty(protocol.packed_bytes(n * 2, layout), dtype=torch.uint8, device=DEV)

            def step():
                protocol.pack(raw, 1, layout, out=msg)
                protocol.unpack(msg, back, 1, layout, bad_flags=bad)
            ms = time_ms(step, reps * (20 if n < 1 << 20 else 1))
            ok = bool(torch.equal(raw, back)) and int(bad.item()) == 0
            emit(config=1, op="pack + unpack", layout=name, bytes=n * 2, us=round(ms * 1e3, 2),
                 ok=ok, hbm_bytes=2 * (n * 2 + msg.numel()))
        del raw, back, msg


def config2(reps: int) -> None:
    n = 134217728
    g = torch.Generator(device=DEV).manual_seed(1)
    src = torch.randn(n, generator=g, device=DEV, dtype=torch.float32).to(torch.float16)
    dst = torch.zeros_like(src)
    S = n * 2
    for name, proto in (("ll128", 0), ("simple", 1)):
        for label, slots in geometries("8x512KiB", (8, 512 * 1024)):
            comm = comm_for(2, proto, slots, waves_per_rank=512 if slots else None)

            def step():
                with comm.rank(0):
                    sendrecv_buffer.send(src, 1, comm)
                with comm.rank(1):
                    sendrecv_buffer.recv(dst, 0, comm)
                sendrecv_buffer.sync(comm)

            dst.zero_()
            step()
            comm.check()
            ok = torch.equal(dst.view(torch.int16), src.view(torch.int16))
            ms = time_ms(step, reps)
            emit(config=2, op="sendrecv", protocol=name, staging=label, bytes=S, ms=round(ms, 4),
                 alg_gbps=round(4 * S / ms / 1e6, 1), hbm_bytes=2 * S,
                 algbw_gbps=round(S / ms / 1e6, 1), ok=ok, grid=comm.last_grid)
    comm = VirtualComm(world_size=2, device=DEV)

    def direct():
        with comm.rank(0):
            sendrecv_direct.send(src, 1, comm)
        with comm.rank(1):
            sendrecv_direct.recv(dst, 0, profile=False, comm=comm)

    dst.zero_()
    direct()
    torch.cuda.synchronize()
    ok = torch.equal(dst.view(torch.int16), src.view(torch.int16))
    ms = time_ms(direct, reps)
    emit(config=2, op="sendrecv_direct", protocol="simple copy", bytes=S, ms=round(ms, 4),
         alg_gbps=round(2 * S / ms / 1e6, 1), hbm_bytes=2 * S, algbw_gbps=round(S / ms / 1e6, 1), ok=ok)


def config3(reps: int) -> None:
    world, n = 8, 33554432
    g = torch.Generator(device=DEV).manual_seed(2)
    root = (torch.rand(n, generator=g, device=DEV) * 8 - 4).to(torch.float16)
    bufs = [root.clone() if r == 0 else torch.zeros_like(root) for r in range(world)]
    S = n * 2
    for name, proto in (("ll128", 0), ("simple", 1)):
        for label, slots in geometries("8x512KiB", (8, 512 * 1024)):
            comm = comm_for(world, proto, slots, waves_per_rank=512 if slots else None)
            for b in bufs[1:]:
                b.zero_()

            def step():
                comm.run(lambda r: broadcast(bufs[r], 0, comm))

            step()
            comm.check()
            ok = all(torch.equal(b.view(torch.int16), root.view(torch.int16)) for b in bufs)
            ms = time_ms(step, reps)
            emit(config=3, op="broadcast", protocol=name, staging=label, world=world, bytes=S,
                 ms=round(ms, 4), alg_gbps=round((3 * world - 2) * S / ms / 1e6, 1),
                 hbm_bytes=world * S, algbw_gbps=round(S / ms / 1e6, 1), ok=ok, grid=comm.last_grid)


def fold_device(rows: list, order: list[int]) -> torch.Tensor:
    acc = rows[order[0]].clone()
    for r in order[1:]:
        acc = primitive.Sum(rows[r].contiguous(), acc)
    return acc


def config4(reps: int) -> None:
    world, n_total = 8, 33554432
    n = n_total // world
    for dt in ("f16", "bf16", "f32"):
        orig = []
        for r in range(world):
            g = torch.Generator(device=DEV).manual_seed(3000 + r)
            orig.append(torch.randn(world, n, generator=g, device=DEV, dtype=torch.float32)
                        .to(TDT[dt]))
        S = n_total * orig[0].element_size()
        for label, slots in geometries("8x1MiB", (8, 1 << 20)):
            comm = comm_for(world, 0, slots, waves_per_rank=512 if slots else None)
            bufs = [o.clone() for o in orig]

            def rs():
                comm.run(lambda r: reducescatter(bufs[r], comm))

            rs()
            comm.check()
            ok = all(torch.equal(bufs[c][c].view(torch.uint8),
                                 fold_device([orig[r][c] for r in range(world)],
                                             [(c + k) % world for k in range(world)]).view(torch.uint8))
                     for c in range(world))
            ms = time_ms(rs, reps)
            emit(config=4, op="reducescatter", dtype=dt, staging=label, world=world, bytes=S,
                 ms=round(ms, 4), alg_gbps=round((3 * world + 1) * S / ms / 1e6, 1),
                 hbm_bytes=(world + 1) * S, algbw_gbps=round(S / ms / 1e6, 1), ok=ok, grid=comm.last_grid)
            flat = [o.reshape(-1).clone() for o in orig]

            def rd():
                comm.run(lambda r: reduce(flat[r], 0, comm))

            rd()
            comm.check()
            ok = torch.equal(flat[0].view(torch.uint8),
                             fold_device([o.reshape(-1) for o in orig], list(range(world)))
                             .view(torch.uint8))
            ms = time_ms(rd, reps)
            emit(config=4, op="reduce", dtype=dt, staging=label, world=world, bytes=S,
                 ms=round(ms, 4), alg_gbps=round((3 * world + 1) * S / ms / 1e6, 1),
                 hbm_bytes=(world + 1) * S, algbw_gbps=round(S / ms / 1e6, 1), ok=ok, grid=comm.last_grid)


def config5(reps: int, max_log2: int, only_log2=()) -> None:
    world = 8
    for name, proto in (("ll128", 0), ("simple", 1)):
        comms = {label: comm_for(world, proto, slots, waves_per_rank=512 if slots else None)
                 for label, slots in geometries("8x512KiB", (8, 512 * 1024))}
        for log2 in (only_log2 or range(9, max_log2 + 1)):
            shard = 1 << log2
            n = shard // 2
            bufs = []
            for r in range(world):
                g = torch.Generator(device=DEV).manual_seed(4 + r)
                b = torch.zeros(world, n, device=DEV, dtype=torch.float16)
                b[r] = (torch.rand(n, generator=g, device=DEV) * 2 - 1).to(torch.float16)
                bufs.append(b)
            want = torch.stack([bufs[r][r] for r in range(world)])
            for label, comm in comms.items():
                def step():
                    comm.run(lambda r: allgather(bufs[r], comm))

                step()
                comm.check()
                ok = all(torch.equal(b.view(torch.int16), want.view(torch.int16)) for b in bufs)
                # launch straight from a prepared descriptor: leaves out the
                # per-rank Python bookkeeping, which would dominate small sizes
                ptrs = {r: bufs[r].data_ptr() for r in range(world)}
                d = comm.make_op(_lib.OP_ALLGATHER, _lib.BYTES, shard, ptrs, ptrs,
                                 list(range(world)) + [0], row_stride=shard)
                ms = time_ms(lambda: comm.launch(d), (reps if log2 < 24 else max(2, reps // 2)) * 4)
                comm.check()
                S = world * shard
                emit(config=5, op="allgather", protocol=name, staging=label, world=world,
                     shard_bytes=shard, us=round(ms * 1e3, 2),
                     alg_gbps=round((3 * world - 2) * S / ms / 1e6, 1), hbm_bytes=world * S,
                     busbw_gbps=round(shard * (world - 1) / ms / 1e6, 1), ok=ok)
                if label == "tuned" and proto == 0 and log2 in (16, 20, 23, 27):
                    # the temporal schedule (6_allgather.py:25-77): row after row
                    # through one pipeline; same bytes
                    for b in bufs:
                        b.zero_()
                    for r in range(world):
                        bufs[r][r] = want[r]
                    td = comm.make_op(_lib.OP_ALLGATHER_TEMPORAL, _lib.BYTES, shard, ptrs, ptrs,
                                      list(range(world)) + [0], row_stride=shard,
                                      protocol=_lib.PROTO_LL128)
                    comm.launch(td)
                    comm.check()
                    tok = all(torch.equal(b.view(torch.int16), want.view(torch.int16)) for b in bufs)
                    tms = time_ms(lambda: comm.launch(td), (reps if log2 < 24 else max(2, reps // 2)) * 4)
                    comm.check()
                    emit(config=5, op="allgather", protocol=name, staging="tuned, temporal",
                         world=world, shard_bytes=shard, us=round(tms * 1e3, 2),
                         alg_gbps=round((3 * world - 2) * S / tms / 1e6, 1), hbm_bytes=world * S,
                         busbw_gbps=round(shard * (world - 1) / tms / 1e6, 1), ok=tok)
                if label == "tuned" and log2 <= 16 and log2 % 2 == 1:
                    # the same launch as 20 nodes of a HIP graph (epoch in device
                    # memory, advanced by a small kernel in front of every launch):
                    # what the device needs once the host is out of the way
                    gcomm = VirtualComm(world_size=world, device=DEV, protocol=proto,
                                        device_epoch=True)
                    gd = gcomm.make_op(_lib.OP_ALLGATHER, _lib.BYTES, shard, ptrs, ptrs,
                                       list(range(world)) + [0], row_stride=shard)
                    side = torch.cuda.Stream(device=DEV)
                    with torch.cuda.stream(side):
                        gcomm.launch(gd)
                    side.synchronize()
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph, stream=side):
                        for _ in range(20):
                            gcomm.launch(gd)
                    gms = time_ms(graph.replay, reps * 2) / 20
                    gcomm.check()
                    gok = all(torch.equal(b.view(torch.int16), want.view(torch.int16)) for b in bufs)
                    emit(config=5, op="allgather", protocol=name, staging="tuned, graph of 20",
                         world=world, shard_bytes=shard, us=round(gms * 1e3, 2), ok=gok)
            del bufs


def allreduce_bench(reps: int) -> None:
    """The reference's planned 8_allreduce: 8 ranks x 256 MiB fp16, as a
    reduce-scatter launch followed by an allgather launch (the default) and as
    one pass round the ring.  Payload bytes (6N - 4) S for the one pass: per
    chunk N own-row reads, 2N - 2 staging writes and reads, N result writes;
    the same figure is used for both so that the rates compare."""
    from mintccl_amd.allreduce import allreduce
    world = 8
    for n in (33554432, 134217728):
        orig = []
        for r in range(world):
            g = torch.Generator(device=DEV).manual_seed(3000 + r)
            orig.append(torch.randn(n, generator=g, device=DEV, dtype=torch.float32)
                        .to(torch.float16))
        S = n * 2
        for name, proto, fused in (("ll128", 0, False), ("ll128", 0, True), ("simple", 1, False),
                                   ("simple", 1, True)):
            comm = comm_for(world, proto, None)
            bufs = [o.clone() for o in orig]

            def step():
                comm.run(lambda r: allreduce(bufs[r], comm, fused=fused))

            step()
            comm.check()
            row = n // world
            ok = True
            for c in range(world):
                want = fold_device([o[c * row:(c + 1) * row] for o in orig],
                                   [(c + k) % world for k in range(world)])
                ok = ok and all(torch.equal(b[c * row:(c + 1) * row].view(torch.int16),
                                            want.view(torch.int16)) for b in bufs)
            ms = time_ms(step, reps)
            emit(config="next", op="allreduce", protocol=name,
                 mode="one pass" if fused else "reducescatter + allgather", staging="tuned",
                 world=world, bytes=S, ms=round(ms, 4), alg_gbps=round((6 * world - 4) * S / ms / 1e6, 1),
                 hbm_bytes=2 * world * S, algbw_gbps=round(S / ms / 1e6, 1),
                 busbw_gbps=round(2 * (world - 1) / world * S / ms / 1e6, 1), ok=ok,
                 grid=comm.last_grid)
        del orig


def alltoall_bench(reps: int) -> None:
    """The reference's planned 9_alltoall: 8 ranks, 64 and 256 MiB fp16 per
    rank, every row straight into its destination's staging and out again
    (per rank S read, S staged, S taken out of staging, S written: 4 N S)."""
    from mintccl_amd.alltoall import alltoall
    world = 8
    for n_total in (33554432, 134217728):
        n = n_total // world
        bufs = []
        for r in range(world):
            g = torch.Generator(device=DEV).manual_seed(90 + r)
            bufs.append(torch.randn(world, n, generator=g, device=DEV, dtype=torch.float32)
                        .to(torch.float16))
        outs = [torch.zeros_like(b) for b in bufs]
        S = n_total * 2
        for name, proto in (("ll128", 0), ("simple", 1)):
            comm = comm_for(world, proto, None)

            def step():
                comm.run(lambda r: alltoall(bufs[r], outs[r], comm))

            for o in outs:
                o.zero_()
            step()
            comm.check()
            ok = all(torch.equal(outs[d][s].view(torch.int16), bufs[s][d].view(torch.int16))
                     for d in range(world) for s in range(world))
            ms = time_ms(step, reps)
            emit(config="next", op="alltoall", protocol=name, staging="tuned", world=world, bytes=S,
                 ms=round(ms, 4), alg_gbps=round(4 * world * S / ms / 1e6, 1),
                 hbm_bytes=2 * world * S, algbw_gbps=round(S / ms / 1e6, 1), ok=ok,
                 grid=comm.last_grid)
        del bufs, outs


def tree_bench(reps: int, log2s=(10, 14, 17, 20, 23, 26)) -> None:
    """Broadcast and reduce over the binary tree (3 hops deep for 8 ranks)
    beside the ring (7 / 8 hops), 8 ranks, from 1 KiB to 64 MiB per rank,
    launched from prepared descriptors; checked against the device adder folded
    in the tree's / the ring's order."""
    from mintccl_amd import primitive
    world, root = 8, 0
    comm = comm_for(world, 0)
    ring = list(range(world)) + [0]
    for log2 in log2s:
        nbytes = 1 << log2
        n = nbytes // 2
        g = torch.Generator(device=DEV).manual_seed(9)
        src = [(torch.rand(n, generator=g, device=DEV) * 2 - 1).to(torch.float16) for _ in range(world)]

        def tree_sum(h: int) -> torch.Tensor:
            acc = src[h].clone()
            for c in (2 * h + 1, 2 * h + 2):
                if c < world:
                    acc = primitive.Sum(acc, tree_sum(c))
            return acc

        want = {"tree": tree_sum(0), "ring": fold_device(src, list(range(world)))}
        bufs = [x.clone() for x in src]
        ptrs = {r: bufs[r].data_ptr() for r in range(world)}
        for topo, rd, bc in (("ring", _lib.OP_REDUCE, _lib.OP_BROADCAST),
                             ("tree", _lib.OP_TREE_REDUCE, _lib.OP_TREE_BROADCAST)):
            for b, x in zip(bufs, src):
                b.copy_(x)
            d = comm.make_op(rd, _lib.F16, nbytes, ptrs, {root: ptrs[root]}, ring, root=root,
                             protocol=_lib.PROTO_LL128)
            comm.launch(d)
            comm.check()
            ok = torch.equal(bufs[root], want[topo]) and all(
                torch.equal(bufs[r], src[r]) for r in range(1, world))
            # (timed launches keep adding into the root's buffer: the values no longer matter)
            ms = time_ms(lambda: comm.launch(d), reps * 4)
            comm.check()
            emit(config="tree", op="reduce", topology=topo, world=world, bytes=nbytes,
                 us=round(ms * 1e3, 2), hbm_bytes=(world + 1) * nbytes, ok=ok, grid=comm.last_grid)
            d = comm.make_op(bc, _lib.BYTES, nbytes, {root: ptrs[root]},
                             {r: p for r, p in ptrs.items() if r != root}, ring, root=root,
                             protocol=_lib.PROTO_LL128)
            for b in bufs[1:]:
                b.zero_()
            comm.launch(d)
            comm.check()
            ok = all(torch.equal(b, bufs[root]) for b in bufs)
            ms = time_ms(lambda: comm.launch(d), reps * 4)
            comm.check()
            emit(config="tree", op="broadcast", topology=topo, world=world, bytes=nbytes,
                 us=round(ms * 1e3, 2), hbm_bytes=world * nbytes, ok=ok, grid=comm.last_grid)


def hypercube_bench(reps: int, log2s=(14, 20, 26)) -> None:
    """Reduce-scatter and allgather over the hypercube (3 exchanges for 8
    ranks) beside the ring (7 hops), 8 ranks, 16 KiB to 64 MiB per rank,
    launched from prepared descriptors; the reduce-scatter is checked against
    the device adder folded in the hypercube's / the ring's order, the
    allgather against the rows it gathers."""
    from mintccl_amd import hypercube, primitive
    world = 8
    comm = comm_for(world, 0)
    ring = list(range(world)) + [0]
    for log2 in log2s:
        nbytes = 1 << log2
        row = nbytes // world
        n = row // 2
        g = torch.Generator(device=DEV).manual_seed(10)
        src = [(torch.rand(world, n, generator=g, device=DEV) * 2 - 1).to(torch.float16)
               for _ in range(world)]

        def cube_sum(tree, r: int) -> torch.Tensor:
            if isinstance(tree, int):
                return src[tree][r].clone()
            return primitive.Sum(cube_sum(tree[0], r), cube_sum(tree[1], r))

        want = {"hypercube": [cube_sum(hypercube.order(world, r), r) for r in range(world)],
                "ring": [fold_device([x[r] for x in src], [(r + i) % world for i in range(world)])
                         for r in range(world)]}
        bufs = [x.clone() for x in src]
        ptrs = {r: bufs[r].data_ptr() for r in range(world)}
        for topo, rs, ag in (("ring", _lib.OP_REDUCESCATTER, _lib.OP_ALLGATHER),
                             ("hypercube", _lib.OP_HYPERCUBE_REDUCESCATTER,
                              _lib.OP_HYPERCUBE_ALLGATHER)):
            for b, x in zip(bufs, src):
                b.copy_(x)
            d = comm.make_op(rs, _lib.F16, row, ptrs, ptrs, ring, row_stride=row,
                             protocol=_lib.PROTO_LL128)
            comm.launch(d)
            comm.check()
            ok = all(torch.equal(bufs[r][r], want[topo][r]) for r in range(world))
            # (timed launches keep adding into row r of rank r: the values no longer matter)
            ms = time_ms(lambda: comm.launch(d), reps * 4)
            comm.check()
            emit(config="hypercube", op="reducescatter", topology=topo, world=world, bytes=nbytes,
                 us=round(ms * 1e3, 2), hbm_bytes=(world + 1) * nbytes, ok=ok, grid=comm.last_grid)
            for r, b in enumerate(bufs):
                b.zero_()
                b[r].copy_(src[r][r])
            d = comm.make_op(ag, _lib.BYTES, row, ptrs, ptrs, ring, row_stride=row,
                             protocol=_lib.PROTO_LL128)
            comm.launch(d)
            comm.check()
            ok = all(torch.equal(b[c], src[c][c]) for b in bufs for c in range(world))
            ms = time_ms(lambda: comm.launch(d), reps * 4)
            comm.check()
            emit(config="hypercube", op="allgather", topology=topo, world=world, bytes=nbytes,
                 us=round(ms * 1e3, 2), hbm_bytes=world * nbytes, ok=ok, grid=comm.last_grid)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--staging", choices=("both", "reference", "tuned"), default="both")
    ap.add_argument("--quick", action="store_true", help="fewer repetitions, sweep to 16 MiB")
    ap.add_argument("--only", type=int, default=0,
                    help="run one config (1..5; 8 = allreduce; 9 = alltoall; 10 = tree against ring; "
                         "11 = hypercube against ring)")
    ap.add_argument("--shard-log2", default="",
                    help="config 5: only these shard sizes (log2 of bytes, comma separated)")
    ap.add_argument("--tree-log2", default="10,14,17,20,23,26",
                    help="config 10: log2 of the message sizes (bytes per rank)")
    ap.add_argument("--cube-log2", default="14,17,20,23,26",
                    help="config 11: log2 of the message sizes (bytes per rank)")
    args = ap.parse_args()
    global STAGING
    STAGING = ("reference", "tuned") if args.staging == "both" else (args.staging,)
    reps = 3 if args.quick else 8
    torch.cuda.set_device(DEV)
    if args.only in (0, 1):
        config1(reps)
    if args.only in (0, 2):
        config2(reps)
    if args.only in (0, 3):
        config3(reps)
    if args.only in (0, 4):
        config4(reps)
    if args.only in (0, 5):
        config5(reps, 24 if args.quick else 27,
                tuple(int(x) for x in args.shard_log2.split(",") if x))
    if args.only in (0, 8):
        allreduce_bench(reps)
    if args.only in (0, 9):
        alltoall_bench(reps)
    if args.only in (0, 10):
        tree_bench(reps, tuple(int(x) for x in args.tree_log2.split(",")))
    if args.only in (0, 11):
        hypercube_bench(reps, tuple(int(x) for x in args.cube_log2.split(",")))
    return 0


if __name__ == "__main__":
    sys.exit(main())
