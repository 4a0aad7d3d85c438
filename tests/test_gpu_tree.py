"""GPU parity of broadcast / reduce over a binary tree against the oracle
(``oracle.ring.tree_reduce``; a broadcast is bit-exact copies), through the
operator surface and the C ABI.  The reference only plans these
(README.md:52-55): the order of a node's additions, (own + first subtree) +
second subtree, is pinned by the hand-computed values below."""
import numpy as np
import pytest
import torch

from oracle import ring
from tests.helpers import TORCH_DT, as_bytes, normal

pytestmark = pytest.mark.gpu

WORLDS = [2, 3, 4, 5, 7, 8]


def make_comm(world, **kw):
    from mintccl_amd.common import VirtualComm
    kw.setdefault("spin_budget", 400000)
    return VirtualComm(world_size=world, **kw)


def run_reduce(comm, bufs, root):
    from mintccl_amd.tree import reduce
    comm.run(lambda r: reduce(bufs[r], root, comm))
    comm.check()


def run_broadcast(comm, bufs, root):
    from mintccl_amd.tree import broadcast
    comm.run(lambda r: broadcast(bufs[r], root, comm))
    comm.check()


def same(bufs, want) -> bool:
    return all(np.array_equal(as_bytes(b), w) for b, w in zip(bufs, want))


@pytest.mark.parametrize("world", WORLDS)
@pytest.mark.parametrize("root", [0, 1])
@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
def test_tree_reduce(dev, world, root, dt):
    n = 70001
    host = [normal(n, 5000 + r, TORCH_DT[dt]) for r in range(world)]
    bufs = [h.to(dev) for h in host]
    comm = make_comm(world)
    run_reduce(comm, bufs, root)
    assert same(bufs, ring.tree_reduce([as_bytes(h) for h in host], root, dt))


@pytest.mark.parametrize("world", [3, 5, 8])
@pytest.mark.parametrize("n", [1, 7, 479, 480, 481, 4096, 100003])
def test_tree_reduce_ragged_sizes_small_slots(dev, world, n):
    # many steps through two small slots: every credit word is waited for
    host = [normal(n, 5100 + r, torch.float16) for r in range(world)]
    bufs = [h.to(dev) for h in host]
    comm = make_comm(world, buff_size_=2 * 2 * 16 * 1024, nslots=2, waves_per_rank=16)
    root = world - 1
    run_reduce(comm, bufs, root)
    assert same(bufs, ring.tree_reduce([as_bytes(h) for h in host], root, "f16"))


def test_tree_reduce_order_by_hand(dev):
    """2048 has an ulp of 2 in binary16, so where the ones are added shows."""
    def run(values, world, root=0):
        bufs = [torch.full((1000,), v, dtype=torch.float16, device=dev) for v in values]
        comm = make_comm(world)
        run_reduce(comm, bufs, root)
        out = bufs[root].cpu()
        assert bool((out == out[0]).all())
        return float(out[0])
    assert run([2048.0, 1.0, 1.0], 3) == 2048.0          # (2048 + 1) + 1; (1 + 1) + 2048 = 2050
    assert run([2048.0, 1.0, 1.5], 3) == 2050.0          # first child first
    assert run([2048.0, 1.5, 1.0], 3) == 2052.0
    # five nodes: (2048 + ((1 + 1) + 0)) + 0 = 2050; the ring's order gives 2048
    assert run([2048.0, 1.0, 0.0, 1.0, 0.0], 5) == 2050.0
    # root 1 heads the node order 1, 2, 3, 4, 0, which carries 2048, 1, 0, 0, 1: node 1
    # (rank 2) passes up (1 + 0) + 1 = 2, the root stores (2048 + 2) + 0; the ring from
    # rank 1 loses both ones
    assert run([1.0, 2048.0, 1.0, 0.0, 0.0], 5, root=1) == 2050.0


@pytest.mark.parametrize("world", WORLDS)
@pytest.mark.parametrize("nbytes", [1, 7, 960, 961, 1 << 20, (1 << 20) + 3])
def test_tree_broadcast_bytes(dev, world, nbytes):
    root = world - 1
    g = torch.Generator().manual_seed(nbytes)
    host = [torch.randint(0, 256, (nbytes,), dtype=torch.uint8, generator=g) for _ in range(world)]
    bufs = [h.to(dev) for h in host]
    comm = make_comm(world)
    run_broadcast(comm, bufs, root)
    for b in bufs:
        assert torch.equal(b.cpu(), host[root])


@pytest.mark.parametrize("policy", [(0, 0), (1, 0), (1, 2)])
def test_tree_policies_and_placements(dev, policy):
    placement, cache = policy
    world, n = 8, 300007
    comm = make_comm(world, placement=placement, cache_policy=cache, buff_size_=3 * 2 * 64 * 1024,
                     nslots=3, waves_per_rank=64)
    host = [normal(n, 5200 + r, torch.float16) for r in range(world)]
    bufs = [h.to(dev) for h in host]
    run_reduce(comm, bufs, 5)
    assert same(bufs, ring.tree_reduce([as_bytes(h) for h in host], 5, "f16"))
    run_broadcast(comm, bufs, 5)
    want = ring.tree_reduce([as_bytes(h) for h in host], 5, "f16")[5]
    for b in bufs:
        assert np.array_equal(as_bytes(b), want)


def test_tree_over_a_permuted_ring(dev):
    from mintccl_amd import topology
    world, n = 5, 50001
    comm = make_comm(world)
    comm.topology = topology.uniform_topology(world)
    comm._ring_cache = (comm.topology, [0, 2, 1, 3, 4, 0])
    host = [normal(n, 5300 + r, torch.float16) for r in range(world)]
    bufs = [h.to(dev) for h in host]
    run_reduce(comm, bufs, 1)
    assert same(bufs, ring.tree_reduce([as_bytes(h) for h in host], 1, "f16", [0, 2, 1, 3, 4, 0]))


def test_tree_64mib_and_back_to_back_launches(dev):
    """A large message through the tuned geometry, twice in a row on the same
    staging (the second launch meets the first one's tags under another epoch),
    then a ring reduce on the same communicator."""
    from mintccl_amd.reduce import reduce as ring_reduce
    world, n = 8, 32 << 20
    comm = make_comm(world)
    g = torch.Generator(device=dev).manual_seed(77)
    src = [torch.empty(n, dtype=torch.float16, device=dev).uniform_(-1, 1, generator=g)
           for _ in range(world)]
    from mintccl_amd import primitive
    for root in (0, 6):
        bufs = [s.clone() for s in src]
        run_reduce(comm, bufs, root)
        order = ring.tree_nodes(ring.identity_ring(world), root)

        def fold(h):
            acc = src[order[h]].clone()
            for c in (2 * h + 1, 2 * h + 2):
                if c < world:
                    acc = primitive.Sum(acc, fold(c))
            return acc
        assert torch.equal(bufs[root], fold(0))
        for r in range(world):
            if r != root:
                assert torch.equal(bufs[r], src[r])
        run_broadcast(comm, bufs, root)
        for r in range(world):
            assert torch.equal(bufs[r], bufs[root])
    bufs = [s.clone() for s in src]
    comm.run(lambda r: ring_reduce(bufs[r], 2, comm))
    comm.check()
    acc = src[2].clone()
    for r in (3, 4, 5, 6, 7, 0, 1):
        acc = primitive.Sum(src[r], acc)
    assert torch.equal(bufs[2], acc)


def test_topology_switch_routes_the_ring_operators_to_the_tree(dev, monkeypatch):
    from mintccl_amd.broadcast import broadcast
    from mintccl_amd.reduce import reduce
    monkeypatch.setenv("MINTCCL_TOPOLOGY", "tree")
    world = 5
    vals = [2048.0, 1.0, 0.0, 1.0, 0.0]
    bufs = [torch.full((4000,), v, dtype=torch.float16, device=dev) for v in vals]
    comm = make_comm(world)
    comm.run(lambda r: reduce(bufs[r], 0, comm))
    comm.check()
    assert float(bufs[0][0]) == 2050.0 and float(bufs[0][-1]) == 2050.0     # the ring gives 2048
    comm.run(lambda r: broadcast(bufs[r], 0, comm))
    comm.check()
    assert all(float(b[17]) == 2050.0 for b in bufs)


def test_tree_self_tests_pass(dev, monkeypatch, capsys):
    from mintccl_amd import selftest
    monkeypatch.setenv("MINTCCL_TEST_MODE", "1")
    monkeypatch.setenv("MINTCCL_TEST_COUNT", str(1 << 20))
    monkeypatch.setenv("ROOT_TEMP", "3")
    assert selftest.main("tree_broadcast") == 0
    assert selftest.main("tree_reduce") == 0
    out = capsys.readouterr().out
    assert out.count("equal: True") == 8 + 1 and "equal: False" not in out


def test_ring_self_tests_follow_the_topology_switch(dev, monkeypatch, capsys):
    """With MINTCCL_TOPOLOGY=tree the reduce self-test compares with the tree's
    order of additions (the operator it runs went up the tree)."""
    from mintccl_amd import selftest
    monkeypatch.setenv("MINTCCL_TEST_MODE", "1")
    monkeypatch.setenv("MINTCCL_TEST_COUNT", str(1 << 18))
    monkeypatch.setenv("MINTCCL_WORLD_SIZE", "5")
    monkeypatch.setenv("MINTCCL_TOPOLOGY", "tree")
    monkeypatch.setenv("MINTCCL_ALLGATHER", "temporal")
    assert selftest.main("reduce") == 0
    assert selftest.main("broadcast") == 0
    assert selftest.main("allgather") == 0
    out = capsys.readouterr().out
    assert "equal: False" not in out and out.count("equal: True") == 1 + 5 + 5

