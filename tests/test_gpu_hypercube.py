"""GPU parity of reduce-scatter / allgather over a hypercube against the oracle
(``oracle.ring.hypercube_reducescatter``; an allgather is bit-exact copies),
through the operator surface and the C ABI.  The reference only plans these
(README.md:52-55): the order of the additions - recursive halving, the partner
across the highest bit first - is this build's definition, pinned by the
hand-computed values below and in ``test_oracle_ring``."""
import numpy as np
import pytest
import torch

from oracle import ring
from tests.helpers import TORCH_DT, as_bytes, rank_rows

pytestmark = pytest.mark.gpu

WORLDS = [2, 4, 8]


def make_comm(world, **kw):
    from mintccl_amd.common import VirtualComm
    kw.setdefault("spin_budget", 400000)
    return VirtualComm(world_size=world, **kw)


def run_reducescatter(comm, bufs):
    from mintccl_amd.hypercube import reducescatter
    comm.run(lambda r: reducescatter(bufs[r], comm))
    comm.check()


def run_allgather(comm, bufs):
    from mintccl_amd.hypercube import allgather
    comm.run(lambda r: allgather(bufs[r], comm))
    comm.check()


def same(bufs, want) -> bool:
    return all(np.array_equal(as_bytes(b), w) for b, w in zip(bufs, want))


@pytest.mark.parametrize("world", WORLDS)
@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
def test_hypercube_reducescatter(dev, world, dt):
    n = 40001
    host = rank_rows(world, n, dt, 6000)
    bufs = [h.to(dev) for h in host]
    comm = make_comm(world)
    run_reducescatter(comm, bufs)
    assert same(bufs, ring.hypercube_reducescatter([as_bytes(h) for h in host], dt))


@pytest.mark.parametrize("world", WORLDS)
@pytest.mark.parametrize("n", [1, 7, 479, 480, 481, 4096, 50003])
def test_hypercube_reducescatter_ragged_sizes_small_slots(dev, world, n):
    # many steps through two small slots: every credit word is waited for
    host = rank_rows(world, n, "f16", 6100)
    bufs = [h.to(dev) for h in host]
    shares = max(1, world - 1)
    comm = make_comm(world, buff_size_=2 * shares * 8 * 1024, nslots=2, waves_per_rank=8 * world)
    run_reducescatter(comm, bufs)
    assert same(bufs, ring.hypercube_reducescatter([as_bytes(h) for h in host], "f16"))


def test_hypercube_order_by_hand(dev):
    """2048 has an ulp of 2 in binary16, so where the small values are added
    shows (the arithmetic is spelt out in test_oracle_ring)."""
    def run(values, world, row):
        bufs = []
        for v in values:
            b = torch.zeros((world, 1000), dtype=torch.float16, device=dev)
            b[row] = v
            bufs.append(b)
        comm = make_comm(world)
        run_reducescatter(comm, bufs)
        out = bufs[row][row].cpu()
        assert bool((out == out[0]).all())
        return float(out[0])
    # (x0 + x2) + (x1 + x3): (2048 + 1.5) + (1 + 0) -> 2052; ring and binary tree give 2050
    assert run([2048.0, 1.0, 1.5, 0.0], 4, 0) == 2052.0
    assert run([1.0, 1.5, 0.0, 2048.0], 4, 3) == 2052.0
    # ((x0 + x4) + (x2 + x6)) + ((x1 + x5) + (x3 + x7)) -> 2056; the ring gives 2052
    assert run([2048.0, 1.0, 1.0, 1.0, 1.5, 1.0, 0.0, 0.0], 8, 0) == 2056.0
    vals = [0.0] * 8
    for part, v in zip((5, 1, 7, 3, 4, 0, 6, 2), (2048.0, 1.5, 1.0, 0.0, 1.0, 1.0, 1.0, 0.0)):
        vals[part] = v
    assert run(vals, 8, 5) == 2056.0


@pytest.mark.parametrize("world", WORLDS)
@pytest.mark.parametrize("nbytes", [1, 7, 960, 961, 1 << 18, (1 << 18) + 3])
def test_hypercube_allgather_bytes(dev, world, nbytes):
    g = torch.Generator().manual_seed(nbytes)
    host = [torch.randint(0, 256, (world, nbytes), dtype=torch.uint8, generator=g)
            for _ in range(world)]
    bufs = [h.to(dev) for h in host]
    comm = make_comm(world)
    run_allgather(comm, bufs)
    assert same(bufs, ring.hypercube_allgather([as_bytes(h) for h in host]))
    assert same(bufs, ring.allgather([as_bytes(h) for h in host]))


@pytest.mark.parametrize("world", [4, 8])
def test_hypercube_allgather_small_slots(dev, world):
    n = 70001
    host = rank_rows(world, n, "f16", 6200)
    bufs = [h.to(dev) for h in host]
    shares = world - 1
    comm = make_comm(world, buff_size_=2 * shares * 8 * 1024, nslots=2, waves_per_rank=8 * world)
    run_allgather(comm, bufs)
    assert same(bufs, ring.allgather([as_bytes(h) for h in host]))


@pytest.mark.parametrize("policy", [(0, 0), (0, 1), (1, 0), (1, 2)])
def test_hypercube_policies_and_placements(dev, policy):
    placement, cache = policy
    world, n = 8, 100003
    comm = make_comm(world, placement=placement, cache_policy=cache,
                     buff_size_=3 * 7 * 16 * 1024, nslots=3, waves_per_rank=128)
    host = rank_rows(world, n, "f16", 6300)
    bufs = [h.to(dev) for h in host]
    run_reducescatter(comm, bufs)
    want = ring.hypercube_reducescatter([as_bytes(h) for h in host], "f16")
    assert same(bufs, want)
    run_allgather(comm, bufs)
    assert same(bufs, ring.allgather(want))


def test_hypercube_over_a_permuted_ring(dev):
    from mintccl_amd import topology
    world, n = 8, 30001
    order = [0, 2, 1, 3, 7, 5, 6, 4, 0]
    comm = make_comm(world)
    comm.topology = topology.uniform_topology(world)
    comm._ring_cache = (comm.topology, order)
    host = rank_rows(world, n, "f16", 6400)
    bufs = [h.to(dev) for h in host]
    run_reducescatter(comm, bufs)
    want = ring.hypercube_reducescatter([as_bytes(h) for h in host], "f16", order)
    assert same(bufs, want)
    # (the order matters: the identity ring's result differs somewhere)
    assert not all(np.array_equal(a, b) for a, b in zip(
        want, ring.hypercube_reducescatter([as_bytes(h) for h in host], "f16")))
    run_allgather(comm, bufs)
    assert same(bufs, ring.allgather(want))


def test_hypercube_64mib_and_back_to_back_launches(dev):
    """A large message through the tuned geometry, twice in a row on the same
    staging (the second launch meets the first one's tags under another epoch),
    then a ring reduce-scatter on the same communicator; checked against torch
    additions in the hypercube's order and, for the allgather that follows,
    through the round trip."""
    from mintccl_amd import hypercube, primitive
    from mintccl_amd.reducescatter import reducescatter as ring_reducescatter
    world, n = 8, (64 << 20) // 2 // 8
    comm = make_comm(world)
    g = torch.Generator(device=dev).manual_seed(78)
    src = [torch.empty(world, n, dtype=torch.float16, device=dev).uniform_(-1, 1, generator=g)
           for _ in range(world)]

    def fold(tree, row):
        if isinstance(tree, int):
            return src[tree][row].clone()
        return primitive.Sum(fold(tree[0], row), fold(tree[1], row))
    for _ in range(2):
        bufs = [s.clone() for s in src]
        run_reducescatter(comm, bufs)
        for r in range(world):
            assert torch.equal(bufs[r][r], fold(hypercube.order(world, r), r))
            for c in range(world):
                if c != r:
                    assert torch.equal(bufs[r][c], src[r][c])
        run_allgather(comm, bufs)
        for r in range(world):
            for c in range(world):
                assert torch.equal(bufs[r][c], bufs[c][c])
    bufs = [s.clone() for s in src]
    comm.run(lambda r: ring_reducescatter(bufs[r], comm))
    comm.check()
    acc = src[2][2].clone()
    for r in (3, 4, 5, 6, 7, 0, 1):
        acc = primitive.Sum(src[r][2], acc)
    assert torch.equal(bufs[2][2], acc)


def test_hypercube_refuses_what_it_cannot_do(dev):
    from mintccl_amd import _lib, hypercube
    from mintccl_amd._ops import ring_of
    comm = make_comm(3)
    buf = torch.zeros(3, 64, dtype=torch.float16, device=dev)
    with comm.rank(0), pytest.raises(ValueError):
        hypercube.reducescatter(buf, comm)
    # the C ABI says the same: a world of 6, the Simple protocol
    comm = make_comm(6)
    ptrs = {r: buf.data_ptr() for r in range(6)}
    d = comm.make_op(_lib.OP_HYPERCUBE_ALLGATHER, _lib.BYTES, 16, ptrs, ptrs, ring_of(comm),
                     row_stride=16, protocol=_lib.PROTO_LL128)
    assert _lib.lib().mint_ring_grid_blocks(d) == _lib.ERR_ARG
    comm = make_comm(4)
    big = torch.zeros(4, 64, dtype=torch.float16, device=dev)
    ptrs = {r: big.data_ptr() for r in range(4)}
    d = comm.make_op(_lib.OP_HYPERCUBE_REDUCESCATTER, _lib.F16, 128, ptrs, ptrs, ring_of(comm),
                     row_stride=128, protocol=_lib.PROTO_SIMPLE)
    assert _lib.lib().mint_ring_grid_blocks(d) == _lib.ERR_ARG


def test_topology_switch_routes_the_ring_operators_to_the_hypercube(dev, monkeypatch):
    from mintccl_amd.allgather import allgather
    from mintccl_amd.reducescatter import reducescatter
    monkeypatch.setenv("MINTCCL_TOPOLOGY", "hypercube")
    world = 4
    bufs = []
    for v in (2048.0, 1.0, 1.5, 0.0):
        b = torch.zeros((world, 4000), dtype=torch.float16, device=dev)
        b[0] = v
        bufs.append(b)
    comm = make_comm(world)
    comm.run(lambda r: reducescatter(bufs[r], comm))
    comm.check()
    assert float(bufs[0][0][0]) == 2052.0 and float(bufs[0][0][-1]) == 2052.0   # the ring gives 2050
    comm.run(lambda r: allgather(bufs[r], comm))
    comm.check()
    assert all(float(b[0][17]) == 2052.0 for b in bufs)


def test_hypercube_self_tests_pass(dev, monkeypatch, capsys):
    from mintccl_amd import selftest
    monkeypatch.setenv("MINTCCL_TEST_MODE", "1")
    monkeypatch.setenv("MINTCCL_TEST_COUNT", str(1 << 20))
    assert selftest.main("hypercube_reducescatter") == 0
    assert selftest.main("hypercube_allgather") == 0
    monkeypatch.setenv("MINTCCL_TOPOLOGY", "hypercube")
    assert selftest.main("reducescatter") == 0
    out = capsys.readouterr().out
    assert out.count("equal: True") == 8 + 8 + 8 and "equal: False" not in out
