"""Seeded random walk over collectives, world sizes, element types, protocols,
placements, cache policies, slot geometries and ragged sizes: every case is
checked bit for bit against the oracle.  Sizes stay small (the oracle answers
in milliseconds); what varies is everything the scheduler, the flow control
and the guarded ends depend on."""
import random

import numpy as np
import pytest
import torch

from oracle import ring
from tests.helpers import TORCH_DT, as_bytes, rank_rows

pytestmark = pytest.mark.gpu

OPS = ["reducescatter", "allgather", "reduce", "broadcast", "allreduce"]


def one_case(rng: random.Random, dev, case: int, long_rows: bool = False):
    from mintccl_amd import _lib
    from mintccl_amd.allgather import allgather
    from mintccl_amd.allreduce import allreduce
    from mintccl_amd.broadcast import broadcast
    from mintccl_amd.common import VirtualComm
    from mintccl_amd.reduce import reduce
    from mintccl_amd.reducescatter import reducescatter

    op = rng.choice(OPS)
    world = rng.choice([2, 3, 4, 5, 6, 7, 8])
    dt = rng.choice(["f16", "bf16", "f32"])
    proto = rng.choice([0, 1])
    place, cp = rng.choice([(0, 0), (0, 1), (1, 0), (1, 2)])
    nslots = rng.choice([1, 2, 3, 5, 8])
    pipes = world * (2 if op == "allreduce" else 1) if op in ("reducescatter", "allgather", "allreduce") else 1
    per_pipe_blocks = rng.choice([1, 2, 3, 4, 6, 8, 12, 16])
    slot = pipes * per_pipe_blocks * 1024
    waves = pipes * rng.choice([d for d in (1, 2, 3, 4, 6, 8, 12, 16) if per_pipe_blocks % d == 0])
    n = rng.choice([1, 7, 239, 480, 481, 959, 1921, 4099, rng.randrange(1, 30000)])
    if long_rows:
        n = rng.randrange(60000, 400000)      # rows of many whole steps
    root = rng.randrange(world)
    shift = rng.choice([0, 0, 1, 3])
    what = f"case {case}: {op} world {world} {dt} proto {proto} place {place} cp {cp} slots {nslots}x{slot} " \
           f"waves {waves} n {n} root {root} shift {shift}"
    comm = VirtualComm(world_size=world, device=dev, buff_size_=nslots * slot, nslots=nslots,
                       waves_per_rank=waves, protocol=proto, placement=place, cache_policy=cp,
                       spin_budget=400000)
    host = rank_rows(world, n, dt, seed0=7000 + 10 * case)
    backing = [torch.zeros(world * n + 8, dtype=TORCH_DT[dt], device=dev) for _ in range(world)]
    bufs = [b[shift: shift + world * n].view(world, n) for b in backing]
    for b, h in zip(bufs, host):
        b.copy_(h)
    raw = [as_bytes(h) for h in host]
    try:
        if op == "reducescatter":
            comm.run(lambda r: reducescatter(bufs[r], comm))
            want = ring.reducescatter(raw, dt)
        elif op == "allgather":
            comm.run(lambda r: allgather(bufs[r], comm))
            want = ring.allgather(raw)
        elif op == "reduce":
            comm.run(lambda r: reduce(bufs[r], root, comm))
            want = ring.reduce(raw, root, dt)
        elif op == "broadcast":
            comm.run(lambda r: broadcast(bufs[r], root, comm))
            want = ring.broadcast(raw, root)
        else:
            fused = rng.random() < 0.5
            what += f" fused {fused}"
            comm.run(lambda r: allreduce(bufs[r].view(-1), comm, fused=fused))
            want = ring.allreduce(raw, dt)
    except _lib.MintError as e:
        if e.code in (_lib.ERR_GEOMETRY, _lib.ERR_RESIDENCY):
            return False, what
        raise AssertionError(f"{what}: {e}") from e
    comm.check()
    for r in range(world):
        assert ring.same_values(as_bytes(bufs[r]), want[r], dt), f"{what}: rank {r} differs"
        assert float(backing[r][:shift].abs().sum()) == 0, f"{what}: wrote before the buffer"
        assert float(backing[r][shift + world * n:].abs().sum()) == 0, f"{what}: wrote behind the buffer"
    return True, what


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6])
def test_random_cases_match_the_oracle(dev, seed):
    rng = random.Random(seed)
    ran = 0
    for case in range(80):
        print(f"seed {seed}", end=" ", flush=True)
        ok, what = one_case(rng, dev, seed * 1000 + case)
        print(what, "" if ok else "(geometry refused)", flush=True)
        ran += ok
    assert ran >= 60


def one_case_of_the_other_walks(rng: random.Random, dev, case: int, long_rows: bool = False):
    """Binary tree and hypercube (LL128 only): the walks beside the ring's."""
    from mintccl_amd import _lib, hypercube, tree
    from mintccl_amd.common import VirtualComm

    op = rng.choice(["tree_reduce", "tree_broadcast", "cube_reducescatter", "cube_allgather"])
    cube = op.startswith("cube")
    world = rng.choice([2, 4, 8] if cube else [2, 3, 4, 5, 6, 7, 8])
    dt = rng.choice(["f16", "bf16", "f32"])
    place, cp = rng.choice([(0, 0), (0, 1), (1, 0), (1, 2)])
    nslots = rng.choice([1, 2, 3, 5, 8])
    shares = max(1, world - 1) if cube else (2 if op == "tree_reduce" else 1)
    per_share_blocks = rng.choice([1, 2, 3, 4, 6, 8, 12, 16])
    slot = shares * per_share_blocks * 1024
    groups = world if cube else 1
    waves = groups * rng.choice([d for d in (1, 2, 3, 4, 6, 8, 12, 16) if per_share_blocks % d == 0])
    n = rng.choice([1, 7, 239, 480, 481, 959, 1921, 4099, rng.randrange(1, 30000)])
    if long_rows:
        n = rng.randrange(60000, 400000)      # rows of many whole steps
    root = rng.randrange(world)
    shift = rng.choice([0, 0, 1, 3])
    what = f"case {case}: {op} world {world} {dt} place {place} cp {cp} slots {nslots}x{slot} " \
           f"waves {waves} n {n} root {root} shift {shift}"
    comm = VirtualComm(world_size=world, device=dev, buff_size_=nslots * slot, nslots=nslots,
                       waves_per_rank=waves, placement=place, cache_policy=cp, spin_budget=400000)
    host = rank_rows(world, n, dt, seed0=9000 + 10 * case)
    backing = [torch.zeros(world * n + 8, dtype=TORCH_DT[dt], device=dev) for _ in range(world)]
    bufs = [b[shift: shift + world * n].view(world, n) for b in backing]
    for b, h in zip(bufs, host):
        b.copy_(h)
    raw = [as_bytes(h) for h in host]
    try:
        if op == "tree_reduce":
            comm.run(lambda r: tree.reduce(bufs[r], root, comm))
            want = ring.tree_reduce(raw, root, dt)
        elif op == "tree_broadcast":
            comm.run(lambda r: tree.broadcast(bufs[r], root, comm))
            want = ring.broadcast(raw, root)
        elif op == "cube_reducescatter":
            comm.run(lambda r: hypercube.reducescatter(bufs[r], comm))
            want = ring.hypercube_reducescatter(raw, dt)
        else:
            comm.run(lambda r: hypercube.allgather(bufs[r], comm))
            want = ring.hypercube_allgather(raw)
    except _lib.MintError as e:
        if e.code in (_lib.ERR_GEOMETRY, _lib.ERR_RESIDENCY):
            return False, what
        raise AssertionError(f"{what}: {e}") from e
    comm.check()
    for r in range(world):
        assert ring.same_values(as_bytes(bufs[r]), want[r], dt), f"{what}: rank {r} differs"
        assert float(backing[r][:shift].abs().sum()) == 0, f"{what}: wrote before the buffer"
        assert float(backing[r][shift + world * n:].abs().sum()) == 0, f"{what}: wrote behind the buffer"
    return True, what


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_tree_and_hypercube_cases_match_the_oracle(dev, seed):
    rng = random.Random(seed)
    ran = 0
    for case in range(80):
        print(f"seed {seed}", end=" ", flush=True)
        ok, what = one_case_of_the_other_walks(rng, dev, seed * 1000 + case)
        print(what, "" if ok else "(geometry refused)", flush=True)
        ran += ok
    assert ran >= 60


@pytest.mark.parametrize("seed", [21, 22])
def test_random_cases_with_long_rows_match_the_oracle(dev, seed):
    """The same walks on rows of many whole steps: the loops that run whole
    steps (ring, Simple, tree and hypercube nodes) under random geometries."""
    rng = random.Random(seed)
    ran = 0
    for case in range(24):
        ok, what = one_case(rng, dev, seed * 1000 + case, long_rows=True)
        print(what, "" if ok else "(geometry refused)", flush=True)
        ran += ok
    for case in range(12):
        ok, what = one_case_of_the_other_walks(rng, dev, seed * 1000 + 100 + case, long_rows=True)
        print(what, "" if ok else "(geometry refused)", flush=True)
        ran += ok
    assert ran >= 24

