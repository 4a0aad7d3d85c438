"""Self-test blocks of the reference scripts, for virtual ranks on one GPU.

The reference verifies itself from the ``if __name__ == "__main__"`` block of
every script, run under ``mpirun`` with ``MINTCCL_TEST_MODE`` set: it performs
the collective, performs it again with ``torch.distributed`` (NCCL) and prints
``equal: True/False`` plus head and tail slices (``4_broadcast.py:104-126``,
``5_reduce.py:123-155``, ``6_allgather.py:160-178``, ``7_reducescatter.py:100-116``,
``3_sendrecv_buffer.py:150-186``).  Here

    MINTCCL_TEST_MODE=1 [MINTCCL_WORLD_SIZE=8] python -m mintccl_amd.reducescatter

does the same with all ranks in one process.  A collective library cannot span
eight ranks on one GPU, so the second result comes from plain torch operations
on the device: a copy for the copying collectives, and for the reductions the
element additions ``own + received`` in ring order (torch adds two fp16 / bf16
values with one rounding, like the kernels), which is the reference's own
order; the distance to an fp32 ``torch.sum`` - the order-free answer a library
would be near to - is printed beside it.  Inputs follow the reference's
(``randn`` / ``random_``, unseeded there; seeded here so that runs repeat).
``ROOT_TEMP``, ``SRC_TEMP`` and ``DST_TEMP`` keep their meaning.
"""
from __future__ import annotations

import os
import sys

import torch

from . import common
from .common import Timer, VirtualComm


def _env_rank(name: str, default: int) -> int:
    return int(os.getenv(name, default))


def _slices(rank: int, ours: torch.Tensor, theirs: torch.Tensor) -> None:
    print(f"# rank {rank} head")
    print(ours.reshape(-1)[:16])
    print(theirs.reshape(-1)[:16])
    print(f"# rank {rank} tail")
    print(ours.reshape(-1)[-16:])
    print(theirs.reshape(-1)[-16:])


def _report(rank: int, ours: torch.Tensor, theirs: torch.Tensor, show: bool) -> bool:
    same = torch.equal(ours.reshape(-1).view(torch.uint8), theirs.reshape(-1).view(torch.uint8))
    print(f"# rank {rank}, equal: {same}")
    if show or not same:
        _slices(rank, ours, theirs)
    if not same:
        bad = (ours.reshape(-1) != theirs.reshape(-1)).nonzero()
        if bad.numel():
            print(f"# rank {rank}, first mismatch at element {int(bad[0])}")    # 5_reduce.py:153-155
    return same


def _ring_fold(rows: list[torch.Tensor], ring: list[int], root: int) -> torch.Tensor:
    """own + received, round the ring from the root (5_reduce.py:70-89)."""
    order = ring[:-1]
    at = order.index(root)
    order = order[at:] + order[:at]
    acc = rows[order[0]].clone()
    for r in order[1:]:
        acc = rows[r] + acc
    return acc


def _run_all(comm: VirtualComm, fn) -> float:
    with Timer(device=True) as t:
        comm.run(fn)
    comm.check()
    return t.elapsed


def _gen(dev) -> torch.Generator:
    return torch.Generator(device=dev).manual_seed(int(os.getenv("MINTCCL_TEST_SEED", 0)))


def sendrecv(module) -> bool:
    """2_sendrecv_indirect.py:170-204 / 3_sendrecv_buffer.py:150-186."""
    comm = VirtualComm()
    dev, n = comm.device, common.test_count()
    src, dst = _env_rank("SRC_TEMP", 0), _env_rank("DST_TEMP", 1 % comm.world_size)
    data = torch.randn(n, device=dev, generator=_gen(dev))
    out = torch.empty(n, device=dev)
    with Timer(device=True):
        with comm.rank(src):
            module.send(data, dst, comm)
        with comm.rank(dst):
            module.recv(out, src, comm)
        for r in range(comm.world_size):
            with comm.rank(r):
                module.sync(comm)
    comm.check()
    return _report(dst, out, data.clone(), True) if common.test_mode() else True


def sendrecv_direct() -> bool:
    """1_sendrecv_direct.py:82-107."""
    from . import sendrecv_direct as m
    comm = VirtualComm()
    dev, n = comm.device, common.test_count()
    src, dst = _env_rank("SRC_TEMP", 0), _env_rank("DST_TEMP", 1 % comm.world_size)
    data = torch.empty(n, device=dev, dtype=torch.float16).random_(generator=_gen(dev))
    out = torch.empty_like(data)
    with comm.rank(src):
        m.send(data, dst, comm)
    with comm.rank(dst):
        m.recv(out, src, comm=comm)
    torch.cuda.synchronize(dev)
    return _report(dst, out, data.clone(), True) if common.test_mode() else True


def broadcast() -> bool:
    """4_broadcast.py:104-126."""
    from .broadcast import broadcast as op
    comm = VirtualComm()
    dev, n, root = comm.device, common.test_count(), _env_rank("ROOT_TEMP", 0)
    g = _gen(dev)
    bufs = [torch.randn(n, device=dev, generator=g) if r == root else torch.empty(n, device=dev)
            for r in range(comm.world_size)]
    want = bufs[root].clone()
    _run_all(comm, lambda r: op(bufs[r], root, comm))
    if not common.test_mode():
        return True
    return all([_report(r, bufs[r], want, r == (root + 1) % comm.world_size)
                for r in range(comm.world_size)])


def allgather() -> bool:
    """6_allgather.py:160-178."""
    from .allgather import allgather as op
    comm = VirtualComm()
    dev, world = comm.device, comm.world_size
    n = common.test_count() // world
    g = _gen(dev)
    bufs = []
    for r in range(world):
        b = torch.zeros(world, n, device=dev)
        b[r].random_(generator=g)
        bufs.append(b)
    want = torch.stack([bufs[r][r] for r in range(world)])
    _run_all(comm, lambda r: op(bufs[r], comm))
    if not common.test_mode():
        return True
    return all([_report(r, bufs[r], want, r == 0) for r in range(world)])


def _reduction_inputs(comm: VirtualComm, shape) -> list[torch.Tensor]:
    g = _gen(comm.device)
    return [torch.randn(shape, device=comm.device, generator=g).to(torch.float16)
            for _ in range(comm.world_size)]


def _order_free_distance(rank: int, ours: torch.Tensor, rows: list[torch.Tensor]) -> None:
    exact = torch.stack([x.float() for x in rows]).sum(0)
    print(f"# rank {rank}, max |ours - fp32 sum|: {float((ours.float() - exact).abs().max()):.4g}")


def reduce() -> bool:
    """5_reduce.py:123-155."""
    from ._ops import ring_of
    from .reduce import reduce as op
    comm = VirtualComm()
    root = _env_rank("ROOT_TEMP", 0)
    bufs = _reduction_inputs(comm, (common.test_count(),))
    inputs = [b.clone() for b in bufs] if common.test_mode() else None
    _run_all(comm, lambda r: op(bufs[r], root, comm))
    if inputs is None:
        return True
    from . import tree
    if tree.topology_env() == "tree":       # the operator went up the binary tree
        want = _tree_fold(inputs, tree.nodes(ring_of(comm), root))
    else:
        want = _ring_fold(inputs, ring_of(comm), root)
    _order_free_distance(root, bufs[root], inputs)
    return _report(root, bufs[root], want, True)


def reducescatter() -> bool:
    """7_reducescatter.py:100-116."""
    from ._ops import ring_of
    from .reducescatter import reducescatter as op
    comm = VirtualComm()
    world = comm.world_size
    bufs = _reduction_inputs(comm, (world, common.test_count() // world))
    inputs = [b.clone() for b in bufs] if common.test_mode() else None
    _run_all(comm, lambda r: op(bufs[r], comm))
    if inputs is None:
        return True
    from . import hypercube, tree
    ring, ok = ring_of(comm), True
    cube = tree.topology_env() == "hypercube"   # the operator halved recursively
    for r in range(world):
        rows = [x[r] for x in inputs]
        if r == 0:
            _order_free_distance(r, bufs[r][r], rows)
        want = (_cube_fold(rows, hypercube.nodes(ring), r) if cube
                else _ring_fold(rows, ring, r))
        ok &= _report(r, bufs[r][r], want, r == 0)
    return ok


def allreduce() -> bool:
    """The self-test the planned 8_allreduce would carry (README.md:23)."""
    from ._ops import ring_of
    from .allreduce import allreduce as op
    comm = VirtualComm()
    world, n = comm.world_size, common.test_count()
    bufs = _reduction_inputs(comm, (n,))
    inputs = [b.clone() for b in bufs] if common.test_mode() else None
    _run_all(comm, lambda r: op(bufs[r], comm))
    if inputs is None:
        return True
    ring = ring_of(comm)
    row = (-(-n * 2 // world) + 15) // 16 * 16 // 2       # elements per chunk (whole 16-byte vectors)
    want = torch.empty_like(inputs[0])
    for c in range(world):
        lo, hi = min(c * row, n), min((c + 1) * row, n)
        if hi > lo:
            want[lo:hi] = _ring_fold([x[lo:hi] for x in inputs], ring, c)
    _order_free_distance(0, bufs[0], inputs)
    return all([_report(r, bufs[r], want, r == 0) for r in range(world)])


def alltoall() -> bool:
    """The self-test the planned 9_alltoall would carry (README.md:24): the
    second opinion is the transpose done with plain torch copies."""
    from .alltoall import alltoall as op
    comm = VirtualComm()
    dev, world = comm.device, comm.world_size
    n = common.test_count() // world
    g = _gen(dev)
    bufs = [torch.empty(world, n, device=dev).random_(generator=g) for _ in range(world)]
    outs = [torch.zeros_like(b) for b in bufs]
    _run_all(comm, lambda r: op(bufs[r], outs[r], comm))
    if not common.test_mode():
        return True
    return all([_report(d, outs[d], torch.stack([bufs[s][d] for s in range(world)]), d == 0)
                for d in range(world)])


def _tree_fold(rows: list[torch.Tensor], order: list[int], h: int = 0) -> torch.Tensor:
    """(own + first subtree) + second subtree, node ``h`` of the tree over ``order``."""
    acc = rows[order[h]].clone()
    for c in (2 * h + 1, 2 * h + 2):
        if c < len(order):
            acc = acc + _tree_fold(rows, order, c)
    return acc


def _cube_fold(rows: list[torch.Tensor], order: list[int], rank: int) -> torch.Tensor:
    """Row of ``rank`` after recursive halving over the cube whose corner i is
    ``order[i]``: the nested additions ``hypercube.order`` names."""
    from . import hypercube

    def fold(tree):
        if isinstance(tree, int):
            return rows[order[tree]].clone()
        return fold(tree[0]) + fold(tree[1])
    return fold(hypercube.order(len(order), order.index(rank)))


def hypercube_reducescatter() -> bool:
    """What 7_reducescatter.py:100-116 checks, over a hypercube (README.md:52-55)."""
    from ._ops import ring_of
    from .hypercube import nodes, reducescatter as op
    comm = VirtualComm()
    world = comm.world_size
    bufs = _reduction_inputs(comm, (world, common.test_count() // world))
    inputs = [b.clone() for b in bufs] if common.test_mode() else None
    _run_all(comm, lambda r: op(bufs[r], comm))
    if inputs is None:
        return True
    order, ok = nodes(ring_of(comm)), True
    for r in range(world):
        rows = [x[r] for x in inputs]
        if r == 0:
            _order_free_distance(r, bufs[r][r], rows)
        ok &= _report(r, bufs[r][r], _cube_fold(rows, order, r), r == 0)
    return ok


def hypercube_allgather() -> bool:
    """What 6_allgather.py:160-178 checks, over a hypercube (README.md:52-55)."""
    from .hypercube import allgather as op
    comm = VirtualComm()
    dev, world = comm.device, comm.world_size
    n = common.test_count() // world
    g = _gen(dev)
    bufs = []
    for r in range(world):
        b = torch.zeros(world, n, device=dev)
        b[r].random_(generator=g)
        bufs.append(b)
    want = torch.stack([bufs[r][r] for r in range(world)])
    _run_all(comm, lambda r: op(bufs[r], comm))
    if not common.test_mode():
        return True
    return all([_report(r, bufs[r], want, r == 0) for r in range(world)])


def tree_broadcast() -> bool:
    """What 4_broadcast.py:104-126 checks, down the binary tree (README.md:52-55)."""
    from .tree import broadcast as op
    comm = VirtualComm()
    dev, n, root = comm.device, common.test_count(), _env_rank("ROOT_TEMP", 0)
    g = _gen(dev)
    bufs = [torch.randn(n, device=dev, generator=g) if r == root else torch.empty(n, device=dev)
            for r in range(comm.world_size)]
    want = bufs[root].clone()
    _run_all(comm, lambda r: op(bufs[r], root, comm))
    if not common.test_mode():
        return True
    return all([_report(r, bufs[r], want, r == (root + 1) % comm.world_size)
                for r in range(comm.world_size)])


def tree_reduce() -> bool:
    """What 5_reduce.py:123-155 checks, up the binary tree (README.md:52-55)."""
    from ._ops import ring_of
    from .tree import nodes, reduce as op
    comm = VirtualComm()
    root = _env_rank("ROOT_TEMP", 0)
    bufs = _reduction_inputs(comm, (common.test_count(),))
    inputs = [b.clone() for b in bufs] if common.test_mode() else None
    _run_all(comm, lambda r: op(bufs[r], root, comm))
    if inputs is None:
        return True
    want = _tree_fold(inputs, nodes(ring_of(comm), root))
    _order_free_distance(root, bufs[root], inputs)
    return _report(root, bufs[root], want, True)


def main(name: str) -> int:
    from . import sendrecv_buffer, sendrecv_indirect
    tests = {"sendrecv_direct": sendrecv_direct,
             "sendrecv_indirect": lambda: sendrecv(sendrecv_indirect),
             "sendrecv_buffer": lambda: sendrecv(sendrecv_buffer),
             "broadcast": broadcast, "reduce": reduce, "allgather": allgather,
             "reducescatter": reducescatter, "allreduce": allreduce, "alltoall": alltoall,
             "tree_broadcast": tree_broadcast, "tree_reduce": tree_reduce,
             "hypercube_reducescatter": hypercube_reducescatter,
             "hypercube_allgather": hypercube_allgather}
    if name == "all":
        world = common.world_size_env()
        if world & (world - 1):         # no hypercube over this many ranks
            tests = {k: fn for k, fn in tests.items() if not k.startswith("hypercube")}
        return 0 if all([fn() for fn in tests.values()]) else 1
    return 0 if tests[name]() else 1


if __name__ == "__main__":
    sys.exit(main(sys.argv[1] if len(sys.argv) > 1 else "all"))
