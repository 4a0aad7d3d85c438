"""GPU parity of the ring collectives against the oracle, through the
operator surface and the C ABI (bit-exact: payloads for the copying ops,
reference fold order for the reductions)."""
import numpy as np
import pytest
import torch

from oracle import ring
from tests.helpers import TORCH_DT, as_bytes, normal, rank_rows, uniform

pytestmark = pytest.mark.gpu


def make_comm(world, **kw):
    from mintccl_amd.common import VirtualComm
    kw.setdefault("spin_budget", 400000)      # ~ a second: a lost line fails, never hangs
    return VirtualComm(world_size=world, **kw)


def run_reducescatter(comm, bufs):
    from mintccl_amd.reducescatter import reducescatter
    comm.run(lambda r: reducescatter(bufs[r], comm))
    comm.check()


def run_allgather(comm, bufs):
    from mintccl_amd.allgather import allgather
    comm.run(lambda r: allgather(bufs[r], comm))
    comm.check()


def run_reduce(comm, bufs, root):
    from mintccl_amd.reduce import reduce
    comm.run(lambda r: reduce(bufs[r], root, comm))
    comm.check()


def run_broadcast(comm, bufs, root):
    from mintccl_amd.broadcast import broadcast
    comm.run(lambda r: broadcast(bufs[r], root, comm))
    comm.check()


def same(bufs, want) -> bool:
    return all(np.array_equal(as_bytes(b), w) for b, w in zip(bufs, want))


WORLDS = [2, 3, 5, 8]
ROW_ELEMS = [1, 8, 479, 480, 481, 4096, 100003]      # ragged, one block, many steps


@pytest.mark.parametrize("world", WORLDS)
@pytest.mark.parametrize("n", ROW_ELEMS)
def test_reducescatter_f16(dev, world, n):
    host = rank_rows(world, n, "f16")
    bufs = [h.to(dev) for h in host]
    comm = make_comm(world, buff_size_=world * 8 * 8192, nslots=8, waves_per_rank=8 * world)
    run_reducescatter(comm, bufs)
    assert same(bufs, ring.reducescatter([as_bytes(h) for h in host], "f16"))


@pytest.mark.parametrize("proto", [0, 1])
@pytest.mark.parametrize("shift", [1, 2, 6, 9])
def test_buffers_and_rows_at_any_byte(dev, proto, shift):
    """Neither the buffers nor the rows of a (world, n) tensor need any
    alignment: buffers carved `shift` elements into an allocation, rows of an
    odd number of elements (many full blocks and a ragged end)."""
    from mintccl_amd.allgather import allgather
    world, n = 4, 3 * 480 * 5 + 7
    host = rank_rows(world, n, "f16")
    backing = [torch.zeros(world * n + 64, dtype=torch.float16, device=dev) for _ in range(world)]
    bufs = [b[shift: shift + world * n].view(world, n) for b in backing]
    for b, h in zip(bufs, host):
        b.copy_(h)
    assert all(b.data_ptr() % 16 == (2 * shift) % 16 for b in bufs)
    comm = make_comm(world, protocol=proto)
    run_reducescatter(comm, bufs)
    assert same(bufs, ring.reducescatter([as_bytes(h) for h in host], "f16"))
    # nothing written outside the buffers
    for b in backing:
        assert int(b[:shift].abs().sum()) == 0 and int(b[shift + world * n:].abs().sum()) == 0
    for b, h in zip(bufs, host):
        b.copy_(h)
    comm.run(lambda r: allgather(bufs[r], comm))
    comm.check()
    assert same(bufs, ring.allgather([as_bytes(h) for h in host]))
    for b in backing:
        assert int(b[:shift].abs().sum()) == 0 and int(b[shift + world * n:].abs().sum()) == 0


@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("proto", [0, 1])
@pytest.mark.parametrize("place,cp", [(0, 0), (1, 0), (0, 1), (1, 2)])
def test_reducescatter_dtypes_protocols_placements(dev, dt, proto, place, cp):
    world, n = 8, 65536 + 8
    host = rank_rows(world, n, dt)
    bufs = [h.to(dev) for h in host]
    comm = make_comm(world, protocol=proto, placement=place, cache_policy=cp)
    run_reducescatter(comm, bufs)
    assert same(bufs, ring.reducescatter([as_bytes(h) for h in host], dt))


@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("threads", [256, 448])
@pytest.mark.parametrize("world,n", [(8, 100003), (8, 480 * 64 * 3), (3, 4099), (5, 7)])
def test_reducescatter_with_own_rows_through_lds(dev, dt, threads, world, n):
    """MINT_FETCH_LDS: one more wavefront per thread block streams the own rows
    into LDS and the wave-channels take them from there.  Same bits as the
    oracle, for thread blocks of 4 and of 7 wave-channels, the tuned geometry
    and small ones with one and with two blocks per wave-channel and step."""
    from mintccl_amd import _lib
    host = rank_rows(world, n, dt, seed0=n)
    want = ring.reducescatter([as_bytes(h) for h in host], dt)
    wpb = threads // 64
    for kw in (dict(), dict(buff_size_=world * 2 * wpb * 2048, nslots=2, waves_per_rank=2 * wpb * world),
               dict(buff_size_=world * 4 * wpb * 2048, nslots=2, waves_per_rank=2 * wpb * world)):
        bufs = [h.to(dev) for h in host]
        comm = make_comm(world, row_fetch=_lib.FETCH_LDS, threads_per_block=threads, **kw)
        run_reducescatter(comm, bufs)
        assert same(bufs, want), kw


@pytest.mark.parametrize("world", [2, 8])
def test_reduce_and_allreduce_with_own_rows_through_lds(dev, world):
    from mintccl_amd import _lib
    from mintccl_amd.allreduce import allreduce
    n = 70001
    host = [normal(n, 50 + r) for r in range(world)]
    raw = [as_bytes(h) for h in host]
    comm = make_comm(world, row_fetch=_lib.FETCH_LDS)
    bufs = [h.to(dev) for h in host]
    run_reduce(comm, bufs, world - 1)
    assert same(bufs, ring.reduce(raw, world - 1, "f16"))
    for fused in (False, True):
        bufs = [h.to(dev) for h in host]
        comm.run(lambda r: allreduce(bufs[r], comm, fused=fused))
        comm.check()
        assert same(bufs, ring.allreduce(raw, "f16"))
    # the copying collectives have no such kernel: the option is ignored
    bufs = [h.to(dev) for h in host]
    run_broadcast(comm, bufs, 0)
    assert same(bufs, ring.broadcast(raw, 0))


@pytest.mark.parametrize("proto", [0, 1])
@pytest.mark.parametrize("world", WORLDS)
@pytest.mark.parametrize("n", [1, 479, 480, 481, 100003])
def test_alltoall(dev, proto, world, n):
    """Row d of rank s arrives as row s of rank d, bit for bit, and the inputs
    are left alone (oracle: the transpose of rows)."""
    from mintccl_amd.alltoall import alltoall
    host = [uniform(world * n, -1.0, 1.0, 70 + r).reshape(world, n) for r in range(world)]
    want = ring.alltoall([as_bytes(h) for h in host])
    for kw in (dict(), dict(buff_size_=world * 8 * 3072, nslots=3, waves_per_rank=2 * 8 * world)):
        bufs = [h.to(dev) for h in host]
        outs = [torch.full_like(b, 7.0) for b in bufs]
        comm = make_comm(world, protocol=proto, **kw)
        comm.run(lambda r: alltoall(bufs[r], outs[r], comm))
        comm.check()
        assert same(outs, want), kw
        assert same(bufs, [as_bytes(h) for h in host])


def test_alltoall_64mib_and_argument_checks(dev):
    from mintccl_amd.alltoall import alltoall
    world, n = 8, 4194304                                   # 8 ranks x 64 MiB fp16
    bufs = []
    for r in range(world):
        g = torch.Generator(device=dev).manual_seed(90 + r)
        bufs.append(torch.randn(world, n, generator=g, device=dev, dtype=torch.float16))
    outs = [torch.zeros_like(b) for b in bufs]
    comm = make_comm(world)
    comm.run(lambda r: alltoall(bufs[r], outs[r], comm))
    comm.check()
    for d in range(world):
        for s in range(world):
            assert torch.equal(outs[d][s].view(torch.int16), bufs[s][d].view(torch.int16)), (d, s)
    with comm.rank(0):
        with pytest.raises(ValueError):
            alltoall(bufs[0], outs[0][:, : n // 2].contiguous(), comm)        # sizes differ
    with pytest.raises(ValueError):
        comm.run(lambda r: alltoall(bufs[r], bufs[(r + 1) % world], comm))    # out is somebody's buff


def test_reducescatter_special_values(dev):
    # overflow to inf, inf - inf, subnormals, signed zeros ride the ring unharmed
    world, n = 4, 960
    vals = torch.tensor([65504.0, -65504.0, 6e-8, -6e-8, 0.0, -0.0, float("inf"), float("-inf"),
                         1.0, 2048.0, 1e-4, 3.0], dtype=torch.float16)
    g = torch.Generator().manual_seed(5)
    host = [vals[torch.randint(0, len(vals), (world * n,), generator=g)].reshape(world, n)
            for _ in range(world)]
    bufs = [h.to(dev) for h in host]
    comm = make_comm(world)
    run_reducescatter(comm, bufs)
    want = ring.reducescatter([as_bytes(h) for h in host], "f16")
    for b, w in zip(bufs, want):
        assert ring.same_values(as_bytes(b), w, "f16")


def test_reducescatter_order_is_the_reference_ring_order(dev):
    # binary16 has ulp 2 at 2048, so 2048 + 1 ties back to 2048 while
    # (1 + 1) + 2048 = 2050: where the large value enters the fold is visible.
    # rows[r][c] = rank r's value for chunk c; chunk c folds in the order
    # c, c+1, ... (7_reducescatter.py:54-73), starting from rank c's own value.
    world, n = 4, 8
    rows = [[2048.0, 1.0, 2048.0, 1.0], [1.0, 1.0, 1.0, 1.0], [1.0, 2048.0, 1.0, 2048.0],
            [1.0, 1.0, 1.0, 1.0]]
    host = [torch.tensor(rows[r], dtype=torch.float16).repeat_interleave(n).reshape(world, n).contiguous()
            for r in range(world)]
    bufs = [h.to(dev) for h in host]
    comm = make_comm(world)
    run_reducescatter(comm, bufs)
    got = [float(bufs[c][c, 0]) for c in range(world)]
    assert got[0] == 2048.0   # 2048, +1 -> 2048, +1 -> 2048, +1 -> 2048
    assert got[1] == 2048.0   # order 1,2,3,0: 1, +2048 -> 2048, +1, +1 (unrotated 0,1,2,3 gives 2052)
    assert got[2] == 2052.0   # order 2,3,0,1: 1, 2, 2050, 2051 -> 2052 (owner-last order gives 2048)
    assert got[3] == 2052.0   # order 3,0,1,2: 1, 2, 3, 2051 -> 2052 (reverse order gives 2048)
    assert same(bufs, ring.reducescatter([as_bytes(h) for h in host], "f16"))


@pytest.mark.parametrize("world", WORLDS)
@pytest.mark.parametrize("root", [0, 1])
@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
def test_reduce(dev, world, root, dt):
    n = 70001
    host = [normal(n, 3000 + r, TORCH_DT[dt]) for r in range(world)]
    bufs = [h.to(dev) for h in host]
    comm = make_comm(world)
    run_reduce(comm, bufs, root)
    assert same(bufs, ring.reduce([as_bytes(h) for h in host], root, dt))


@pytest.mark.parametrize("world", WORLDS)
@pytest.mark.parametrize("nbytes", [1, 7, 960, 961, 1 << 20, (1 << 20) + 3])
@pytest.mark.parametrize("proto", [0, 1])
def test_broadcast_bytes(dev, world, nbytes, proto):
    root = world - 1
    g = torch.Generator().manual_seed(nbytes)
    host = [torch.randint(0, 256, (nbytes,), dtype=torch.uint8, generator=g) for _ in range(world)]
    bufs = [h.to(dev) for h in host]
    comm = make_comm(world, protocol=proto)
    run_broadcast(comm, bufs, root)
    for b in bufs:
        assert torch.equal(b.cpu(), host[root])


@pytest.mark.parametrize("proto", [0, 1])
@pytest.mark.parametrize("policy", [(0, 0), (1, 2)])
def test_an_origin_needs_no_staging(dev, proto, policy):
    """The root of a broadcast and the source of a sendrecv receive nothing:
    the library accepts a descriptor without staging for them and touches none
    (whole steps, a ragged last step and a message shorter than a block)."""
    from mintccl_amd import _lib
    world, root = 4, 3
    comm = make_comm(world, protocol=proto, placement=policy[0], cache_policy=policy[1])
    ring_order = list(range(world)) + [0]
    for nbytes in ((3 << 20) + 5, 100, 960 * 64 * 8):
        g = torch.Generator().manual_seed(nbytes)
        host = [torch.randint(0, 256, (nbytes,), dtype=torch.uint8, generator=g) for _ in range(world)]
        bufs = [h.to(dev) for h in host]
        ptrs = {r: bufs[r].data_ptr() for r in range(world)}
        d = comm.make_op(_lib.OP_BROADCAST, _lib.BYTES, nbytes, {root: ptrs[root]},
                         {r: p for r, p in ptrs.items() if r != root}, ring_order, root=root)
        d.staging[root] = 0
        comm.launch(d)
        comm.check()
        for b in bufs:
            assert torch.equal(b.cpu(), host[root])
        bufs = [h.to(dev) for h in host]
        d = comm.make_op(_lib.OP_SENDRECV, _lib.BYTES, nbytes, {2: bufs[2].data_ptr()},
                         {1: bufs[1].data_ptr()}, [2, 1], route_len=2)
        d.staging[2] = 0
        comm.launch(d)
        comm.check()
        assert torch.equal(bufs[1].cpu(), host[2]) and torch.equal(bufs[0].cpu(), host[0])


@pytest.mark.parametrize("world", WORLDS)
@pytest.mark.parametrize("n", [8, 480, 488, 65536])
@pytest.mark.parametrize("proto", [0, 1])
def test_allgather(dev, world, n, proto):
    host = [uniform(world * n, -1.0, 1.0, 4 + r).reshape(world, n) for r in range(world)]
    bufs = [h.to(dev) for h in host]
    comm = make_comm(world, protocol=proto)
    run_allgather(comm, bufs)
    assert same(bufs, ring.allgather([as_bytes(h) for h in host]))


def run_allgather_temporal(comm, bufs):
    from mintccl_amd.allgather import allgather
    comm.run(lambda r: allgather(bufs[r], comm, schedule="temporal"))
    comm.check()


@pytest.mark.parametrize("world", WORLDS)
@pytest.mark.parametrize("n", [8, 480, 488, 65536])
def test_allgather_temporal_schedule(dev, world, n):
    """6_allgather.py:25-77: the rows go round one after the other; same bytes
    as the spatial schedule."""
    host = [uniform(world * n, -1.0, 1.0, 40 + r).reshape(world, n) for r in range(world)]
    bufs = [h.to(dev) for h in host]
    comm = make_comm(world)
    run_allgather_temporal(comm, bufs)
    assert same(bufs, ring.allgather([as_bytes(h) for h in host]))


@pytest.mark.parametrize("world", [3, 8])
@pytest.mark.parametrize("geometry", [dict(buff_size_=2 * 16 * 1024, nslots=2, waves_per_rank=16),
                                      dict(buff_size_=3 * 64 * 1024, nslots=3, waves_per_rank=32),
                                      dict(buff_size_=5 * 8 * 1024, nslots=5, waves_per_rank=8,
                                           placement=0, cache_policy=0),
                                      dict(buff_size_=2 * 64 * 1024, nslots=2, waves_per_rank=64,
                                           placement=1, cache_policy=2)])
def test_allgather_temporal_many_steps_through_few_slots(dev, world, geometry):
    # 100003 halves per row: 209 blocks, so every row takes several steps and
    # the step count carries on from row to row through the same slots; the
    # link into a row's owner is idle while that row goes round
    n = 100003
    host = [uniform(world * n, -1.0, 1.0, 50 + r).reshape(world, n) for r in range(world)]
    bufs = [h.to(dev) for h in host]
    comm = make_comm(world, **geometry)
    run_allgather_temporal(comm, bufs)
    assert same(bufs, ring.allgather([as_bytes(h) for h in host]))
    # and again on the same staging, then the spatial schedule on top of it
    bufs = [h.to(dev) for h in host]
    run_allgather_temporal(comm, bufs)
    assert same(bufs, ring.allgather([as_bytes(h) for h in host]))
    bufs = [h.to(dev) for h in host]
    run_allgather(comm, bufs)
    assert same(bufs, ring.allgather([as_bytes(h) for h in host]))


def test_allgather_temporal_over_a_permuted_ring_and_by_env(dev, monkeypatch):
    from mintccl_amd import topology
    from mintccl_amd.allgather import allgather
    world, n = 5, 30001
    comm = make_comm(world)
    comm.topology = topology.uniform_topology(world)
    comm._ring_cache = (comm.topology, [0, 2, 4, 1, 3, 0])
    host = [uniform(world * n, -1.0, 1.0, 60 + r).reshape(world, n) for r in range(world)]
    bufs = [h.to(dev) for h in host]
    monkeypatch.setenv("MINTCCL_ALLGATHER", "temporal")
    comm.run(lambda r: allgather(bufs[r], comm))
    comm.check()
    assert same(bufs, ring.allgather([as_bytes(h) for h in host]))
    # one pipeline: 63 blocks per row -> 64 wave-channels per rank, 16 thread blocks each
    assert comm.last_grid == world * 16


def test_allgather_temporal_8_x_8mib(dev):
    world, n = 8, 4 << 20
    g = torch.Generator(device=dev).manual_seed(5)
    bufs = []
    for r in range(world):
        b = torch.zeros(world, n, dtype=torch.float16, device=dev)
        b[r].uniform_(-1, 1, generator=g)
        bufs.append(b)
    want = torch.stack([bufs[r][r] for r in range(world)])
    comm = make_comm(world)
    run_allgather_temporal(comm, bufs)
    for b in bufs:
        assert torch.equal(b, want)


@pytest.mark.parametrize("world", [2, 4, 8])
def test_xcd_local_policy_all_collectives(dev, world):
    # stores that stay in one XCD's L2: every collective, ragged sizes, many
    # steps through 2 small slots
    comm = make_comm(world, placement=1, cache_policy=2, buff_size_=2 * 64 * 1024, nslots=2,
                     waves_per_rank=64)
    n = 200008
    host = rank_rows(world, n, "f16")
    bufs = [h.to(dev) for h in host]
    run_reducescatter(comm, bufs)
    assert same(bufs, ring.reducescatter([as_bytes(h) for h in host], "f16"))
    host = [uniform(world * n, -1.0, 1.0, 4 + r).reshape(world, n) for r in range(world)]
    bufs = [h.to(dev) for h in host]
    run_allgather(comm, bufs)
    assert same(bufs, ring.allgather([as_bytes(h) for h in host]))
    host = [normal(300001, 3000 + r) for r in range(world)]
    bufs = [h.to(dev) for h in host]
    run_reduce(comm, bufs, world - 1)
    assert same(bufs, ring.reduce([as_bytes(h) for h in host], world - 1, "f16"))
    bufs = [h.to(dev) for h in host]
    run_broadcast(comm, bufs, 0)
    for b in bufs:
        assert torch.equal(b.cpu(), host[0])


def test_xcd_local_policy_needs_local_placement(dev):
    with pytest.raises(ValueError):
        make_comm(8, placement=0, cache_policy=2)


def run_allreduce(comm, bufs, fused=False):
    from mintccl_amd.allreduce import allreduce
    comm.run(lambda r: allreduce(bufs[r], comm, fused=fused))
    comm.check()


@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("world", WORLDS)
@pytest.mark.parametrize("n", [1, 7, 8, 63, 64, 4000, 100003, (1 << 20) + 9])
def test_allreduce_f16(dev, world, n, fused):
    # ragged sizes: with few elements some chunks are short or empty; as one
    # pass round the ring, and as a reduce-scatter followed by an allgather
    host = [normal(n, 3000 + r) for r in range(world)]
    bufs = [h.to(dev) for h in host]
    comm = make_comm(world)
    run_allreduce(comm, bufs, fused)
    want = ring.allreduce([as_bytes(h) for h in host], "f16")
    assert same(bufs, want)


@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("dt", ["bf16", "f32"])
@pytest.mark.parametrize("proto,place,cp", [(0, 0, 0), (1, 0, 0), (0, 1, 2), (1, 1, 2)])
def test_allreduce_dtypes_protocols_policies(dev, dt, proto, place, cp, fused):
    world, n = 8, 300001
    host = [normal(n, 3000 + r, TORCH_DT[dt]) for r in range(world)]
    bufs = [h.to(dev) for h in host]
    comm = make_comm(world, protocol=proto, placement=place, cache_policy=cp,
                     buff_size_=3 * 1024 * 1024, nslots=3, waves_per_rank=512)
    run_allreduce(comm, bufs, fused)
    assert same(bufs, ring.allreduce([as_bytes(h) for h in host], dt))


@pytest.mark.parametrize("fused", [False, True])
def test_allreduce_64mib_against_device_fold(dev, fused):
    from mintccl_amd import primitive
    world, n = 8, 33554432          # 64 MiB per rank
    g = torch.Generator(device=dev).manual_seed(11)
    bufs = [torch.randn(n, generator=g, device=dev, dtype=torch.float16) for _ in range(world)]
    orig = [b.clone() for b in bufs]
    comm = make_comm(world)
    run_allreduce(comm, bufs, fused)
    row = n // world
    for c in range(world):
        acc = orig[c][c * row:(c + 1) * row].clone()
        for k in range(1, world):
            acc = primitive.Sum(orig[(c + k) % world][c * row:(c + 1) * row].contiguous(), acc)
        for r in range(world):
            assert torch.equal(bufs[r][c * row:(c + 1) * row].view(torch.int16), acc.view(torch.int16))


def test_permuted_ring(dev):
    # a non-uniform topology whose best ring is not the identity
    from mintccl_amd.topology import find_ring
    world, n = 4, 5000
    fast, slow = 50.0, 5.0
    edges = {(0, 2): fast, (2, 1): fast, (1, 3): fast, (3, 0): fast, (0, 1): slow, (2, 3): slow}
    topo = {i: [] for i in range(world)}
    for (a, b), bw in edges.items():
        topo[a].append((b, bw))
        topo[b].append((a, bw))
    ring_ = find_ring(topo)
    assert ring_ in ([0, 2, 1, 3, 0], [0, 3, 1, 2, 0])
    host = rank_rows(world, n + (-n) % 8, "f16")
    bufs = [h.to(dev) for h in host]
    comm = make_comm(world)
    comm.topology = topo
    run_reducescatter(comm, bufs)
    assert same(bufs, ring.reducescatter([as_bytes(h) for h in host], "f16", ring_))
    host2 = [normal(3001, 50 + r) for r in range(world)]
    bufs2 = [h.to(dev) for h in host2]
    run_reduce(comm, bufs2, 1)
    assert same(bufs2, ring.reduce([as_bytes(h) for h in host2], 1, "f16", ring_))


def test_topology_file_drives_ring_and_route_end_to_end(dev, tmp_path):
    """A non-uniform ``topo.json`` (the reference's file format), written with
    ``save_topology`` and loaded with ``get_topology``: the collectives run
    round the ring it implies, and the deferred send / recv takes the widest
    route - three hops, 0 -> 2 -> 1 -> 3 (bottleneck 47.5 against 24 via rank 1
    alone and 23 via rank 2 alone; ranks 0 and 3 have no direct link)."""
    from mintccl_amd import sendrecv_buffer
    from mintccl_amd.topology import find_ring, find_route, get_topology, save_topology
    world = 4
    links = {(0, 2): 48.0, (2, 1): 47.5, (1, 3): 48.5, (0, 1): 24.0, (2, 3): 23.0}
    topo = {i: [] for i in range(world)}
    for (a, b), bw in links.items():
        topo[a].append((b, bw))
        topo[b].append((a, bw))
    path = str(tmp_path / "topo.json")
    save_topology(topo, path)
    comm = make_comm(world)
    comm.topology = get_topology(path)
    ring_ = find_ring(comm.topology)
    assert ring_ in ([0, 1, 3, 2, 0], [0, 2, 3, 1, 0])          # the two cycles there are
    assert find_route(0, 3, comm.topology) == [0, 2, 1, 3]
    host = rank_rows(world, 20008, "f16")
    bufs = [h.to(dev) for h in host]
    run_reducescatter(comm, bufs)
    assert same(bufs, ring.reducescatter([as_bytes(h) for h in host], "f16", ring_))
    bufs = [h.to(dev) for h in host]
    run_allgather(comm, bufs)
    assert same(bufs, ring.allgather([as_bytes(h) for h in host]))
    src = normal(300007, 9).to(dev)
    dst = torch.zeros_like(src)
    with comm.rank(0):
        sendrecv_buffer.send(src, 3, comm)
    with comm.rank(3):
        sendrecv_buffer.recv(dst, 0, comm)
    sendrecv_buffer.sync(comm)                               # route from the topology
    comm.check()
    assert torch.equal(dst.view(torch.int16), src.view(torch.int16))
    assert comm.last_route == [0, 2, 1, 3]


def test_many_launches_reuse_staging_without_clearing(dev):
    # flags carry a per-launch epoch: stale lines of earlier launches, of other
    # sizes and other collectives, are never mistaken for data
    world = 8
    comm = make_comm(world)
    for i, n in enumerate([4096, 480, 100000, 8, 4096, 52000]):
        host = rank_rows(world, n, "f16", seed0=100 * i)
        bufs = [h.to(dev) for h in host]
        run_reducescatter(comm, bufs)
        assert same(bufs, ring.reducescatter([as_bytes(h) for h in host], "f16"))
        host = [uniform(world * n, -1.0, 1.0, i + r).reshape(world, n) for r in range(world)]
        bufs = [h.to(dev) for h in host]
        run_allgather(comm, bufs)
        assert same(bufs, ring.allgather([as_bytes(h) for h in host]))


def test_epoch_wraps_after_4095_launches(dev):
    # sector tags carry 12 bits of epoch: the communicator clears staging when
    # the counter wraps, so launch 4096 cannot be fooled by launch 1's lines
    from mintccl_amd import _lib
    from mintccl_amd.broadcast import broadcast
    world, n = 4, 2048
    comm = make_comm(world)
    host = [torch.full((n,), float(r + 1), dtype=torch.float16) for r in range(world)]
    bufs = [h.to(dev) for h in host]
    ptrs = {r: bufs[r].data_ptr() for r in range(world)}
    comm.run(lambda r: broadcast(bufs[r], 0, comm))
    d = comm.make_op(_lib.OP_BROADCAST, _lib.BYTES, n * 2, {0: ptrs[0]},
                     {r: ptrs[r] for r in range(1, world)}, [0, 1, 2, 3, 0], root=0)
    for _ in range(_lib.MAX_EPOCH + 5):
        comm.launch(d)
    comm.check()
    assert 1 <= comm.epoch <= 10
    for r in range(world):
        bufs[r].fill_(float(10 + r))
    comm.run(lambda r: broadcast(bufs[r], 2, comm))
    comm.check()
    for b in bufs:
        assert torch.all(b == 12.0)


def test_payload_that_looks_like_credit_words_is_harmless(dev):
    # collectives of different shapes use different slot sizes on the same
    # staging memory; the credit words live at a fixed offset beyond every
    # slot, so payload bytes are never read as credits.  The payload here is
    # 64-bit words (epoch << 32 | huge count) for the epochs that follow.
    from mintccl_amd import sendrecv_buffer
    from mintccl_amd.broadcast import broadcast
    world = 8
    comm = make_comm(world)
    n64 = 1 << 20
    for round_ in range(3):
        words = torch.arange(n64, dtype=torch.int64)
        words = ((comm.epoch + 2 + (words % 3)) << 32) | 0x7FFFFFF0
        src = words.to(dev)
        dst = torch.zeros_like(src)
        with comm.rank(0):
            sendrecv_buffer.send(src, 1, comm)       # 2 positions: large slots
        with comm.rank(1):
            sendrecv_buffer.recv(dst, 0, comm)
        sendrecv_buffer.sync(comm)
        comm.check()
        assert torch.equal(dst, src)
        bufs = [src.clone() if r == 3 else torch.zeros_like(src) for r in range(world)]
        comm.run(lambda r: broadcast(bufs[r], 3, comm))   # 8 positions: small slots
        comm.check()
        for b in bufs:
            assert torch.equal(b, src)
        host = rank_rows(world, 40000, "f16", seed0=round_)
        rs = [h.to(dev) for h in host]
        run_reducescatter(comm, rs)
        assert same(rs, ring.reducescatter([as_bytes(h) for h in host], "f16"))


def test_simple_payload_that_looks_like_ll128_tags_is_harmless(dev):
    # The Simple protocol writes raw payload into the bytes where LL128 keeps
    # its sector tags.  A Simple broadcast whose every 32-bit word is the tag
    # the next LL128 launch expects in step 0 must not make that launch accept
    # stale slots: with the origin withheld, every position still has to run
    # out of patience in step 0 (staging is cleared when LL128 follows Simple).
    from mintccl_amd import _lib
    from mintccl_amd.common import RingTimeout
    world, n32 = 4, 1 << 18
    comm = make_comm(world, spin_budget=2000)
    ring4 = [0, 1, 2, 3, 0]
    bufs = [torch.zeros(n32, dtype=torch.int32, device=dev) for _ in range(world)]
    # the LL128 launch below is the first after the clearing: epoch 1, step 0
    forged = (1 << 20) | 1
    bufs[0].fill_(forged)
    ptrs = {r: bufs[r].data_ptr() for r in range(world)}
    d = comm.make_op(_lib.OP_BROADCAST, _lib.BYTES, n32 * 4, {0: ptrs[0]},
                     {r: ptrs[r] for r in range(1, world)}, ring4, root=0,
                     protocol=_lib.PROTO_SIMPLE)
    comm.launch(d)
    comm.check()
    for b in bufs:
        assert torch.all(b == forged)
    d = comm.make_op(_lib.OP_BROADCAST, _lib.BYTES, n32 * 4, {0: ptrs[0]},
                     {r: ptrs[r] for r in range(1, world)}, ring4, root=0,
                     protocol=_lib.PROTO_LL128, skip_origin=True)
    comm.launch(d)
    assert comm.epoch == 1
    with pytest.raises(RingTimeout, match="step 0"):
        comm.check()


def test_a_lost_producer_times_out_instead_of_hanging(dev):
    from mintccl_amd import _lib
    from mintccl_amd.common import RingTimeout
    world, n = 4, 4096
    comm = make_comm(world, spin_budget=2000)
    bufs = [torch.zeros(n, dtype=torch.float16, device=dev) for _ in range(world)]
    d = comm.make_op(_lib.OP_BROADCAST, _lib.BYTES, n * 2, {0: bufs[0].data_ptr()},
                     {r: bufs[r].data_ptr() for r in range(1, world)}, [0, 1, 2, 3, 0],
                     root=0, skip_origin=True)
    comm.launch(d)
    # two more launches queued behind the one that gives up: they find the abort
    # flag set, give up at their first wait and are counted
    full = comm.make_op(_lib.OP_BROADCAST, _lib.BYTES, n * 2, {0: bufs[0].data_ptr()},
                        {r: bufs[r].data_ptr() for r in range(1, world)}, [0, 1, 2, 3, 0], root=0)
    comm.launch(full)
    comm.launch(full)
    torch.cuda.synchronize(dev)
    st = comm.status.cpu().tolist()
    assert st[0] == 1 and (st[3] & 0xFFFFFFFF) == 1 and (st[3] >> 32) == 2
    with pytest.raises(RingTimeout, match="2 later launch"):
        comm.check()
    # the communicator is usable afterwards
    host = [normal(n, r) for r in range(world)]
    bufs = [h.to(dev) for h in host]
    run_broadcast(comm, bufs, 2)
    for b in bufs:
        assert torch.equal(b.cpu(), host[2])


@pytest.mark.parametrize("world", [2, 3, 5, 6, 7])
def test_large_copying_collectives_over_world_sizes(dev, world):
    """Messages large enough for the full tuned grids, where the origins get
    compute units of their own (a different count for every ring length),
    at odd row sizes: allgather in both schedules, ring and tree broadcast,
    alltoall, sendrecv over one hop."""
    from mintccl_amd import _lib
    n = (3 << 20) + 5 * world + 1                    # bytes per row
    g = torch.Generator().manual_seed(world)
    host = [torch.randint(0, 256, (world, n), dtype=torch.uint8, generator=g) for _ in range(world)]
    ring_order = list(range(world)) + [0]
    comm = make_comm(world)
    want = torch.stack([host[r][r] for r in range(world)])
    for op in (_lib.OP_ALLGATHER, _lib.OP_ALLGATHER_TEMPORAL):
        bufs = [h.to(dev) for h in host]
        ptrs = {r: bufs[r].data_ptr() for r in range(world)}
        d = comm.make_op(op, _lib.BYTES, n, ptrs, ptrs, ring_order, row_stride=n)
        assert d.origin_cus > 0
        comm.launch(d)
        comm.check()
        assert all(torch.equal(b.cpu(), want) for b in bufs)
    root = world - 1
    for op in (_lib.OP_BROADCAST, _lib.OP_TREE_BROADCAST):
        bufs = [h.to(dev) for h in host]
        ptrs = {r: bufs[r].data_ptr() for r in range(world)}
        d = comm.make_op(op, _lib.BYTES, world * n, {root: ptrs[root]},
                         {r: p for r, p in ptrs.items() if r != root}, ring_order, root=root)
        assert d.origin_cus > 0
        comm.launch(d)
        comm.check()
        assert all(torch.equal(b.cpu(), host[root]) for b in bufs)
    bufs = [h.to(dev) for h in host]
    outs = [torch.zeros_like(b) for b in bufs]
    d = comm.make_op(_lib.OP_ALLTOALL, _lib.BYTES, n, {r: bufs[r].data_ptr() for r in range(world)},
                     {r: outs[r].data_ptr() for r in range(world)}, ring_order, row_stride=n)
    assert d.origin_cus > 0
    comm.launch(d)
    comm.check()
    for r in range(world):
        assert torch.equal(outs[r].cpu(), torch.stack([host[q][r] for q in range(world)]))
    d = comm.make_op(_lib.OP_SENDRECV, _lib.BYTES, world * n, {0: bufs[0].data_ptr()},
                     {world - 1: outs[world - 1].data_ptr()}, [0, world - 1], route_len=2)
    assert d.origin_cus > 0
    comm.launch(d)
    comm.check()
    assert torch.equal(outs[world - 1].cpu(), host[0])


def test_origin_cus_that_would_not_be_resident_fall_back_to_the_plain_order(dev):
    """16 of 32 CUs for the origins of an 8-rank allgather with 80 wave-channels
    per (row, hop) would take 9 rounds over the CUs, more than are resident:
    the launch runs in the plain order instead of failing."""
    from mintccl_amd import _lib
    world, n = 8, (2 << 20) + 16
    comm = make_comm(world, buff_size_=2 * 640 * 1024, nslots=2, waves_per_rank=640,
                     placement=1, cache_policy=2, origin_cus=16)
    g = torch.Generator().manual_seed(3)
    host = [torch.randint(0, 256, (world, n), dtype=torch.uint8, generator=g) for _ in range(world)]
    bufs = [h.to(dev) for h in host]
    ptrs = {r: bufs[r].data_ptr() for r in range(world)}
    d = comm.make_op(_lib.OP_ALLGATHER, _lib.BYTES, n, ptrs, ptrs, list(range(world)) + [0], row_stride=n)
    d.flag_epoch = 1                              # (the launch sets its own)
    assert d.origin_cus == 16 and _lib.lib().mint_ring_grid_blocks(d) == 8 * 32 * 9
    comm.launch(d)
    comm.check()
    want = torch.stack([host[r][r] for r in range(world)])
    assert all(torch.equal(b.cpu(), want) for b in bufs)
    # the same for the temporal schedule and the tree at the tuned geometry
    tuned = make_comm(world, origin_cus=20)
    bufs = [h.to(dev) for h in host]
    ptrs = {r: bufs[r].data_ptr() for r in range(world)}
    d = tuned.make_op(_lib.OP_ALLGATHER_TEMPORAL, _lib.BYTES, n, ptrs, ptrs, list(range(world)) + [0],
                      row_stride=n)
    tuned.launch(d)
    tuned.check()
    assert all(torch.equal(b.cpu(), want) for b in bufs)
    bufs = [h.to(dev) for h in host]
    ptrs = {r: bufs[r].data_ptr() for r in range(world)}
    d = tuned.make_op(_lib.OP_TREE_BROADCAST, _lib.BYTES, world * n, {0: ptrs[0]},
                      {r: p for r, p in ptrs.items() if r}, list(range(world)) + [0], root=0)
    tuned.launch(d)
    tuned.check()
    assert all(torch.equal(b.cpu(), host[0]) for b in bufs)


@pytest.mark.parametrize("op", ["broadcast", "allgather", "sendrecv"])
def test_a_spin_limit_of_one_ends_every_wait(dev, op):
    """Large launches at the tuned geometry (origins on compute units of their
    own, fetching ahead, their credit read through the scalar unit) with a
    spin limit of one poll: whoever has to wait gives up at once, every
    wavefront ends, the launch reports a timeout - and the same memory works
    again afterwards."""
    from mintccl_amd import _lib
    from mintccl_amd.common import RingTimeout
    world, n = 8, 4 << 20
    g = torch.Generator().manual_seed(7)
    host = [torch.randint(0, 256, (world, n), dtype=torch.uint8, generator=g) for _ in range(world)]
    bufs = [h.to(dev) for h in host]
    ptrs = {r: bufs[r].data_ptr() for r in range(world)}
    ring_order = list(range(world)) + [0]

    def describe(comm):
        if op == "broadcast":
            return comm.make_op(_lib.OP_BROADCAST, _lib.BYTES, world * n, {0: ptrs[0]},
                                {r: p for r, p in ptrs.items() if r}, ring_order, root=0)
        if op == "allgather":
            return comm.make_op(_lib.OP_ALLGATHER, _lib.BYTES, n, ptrs, ptrs, ring_order, row_stride=n)
        return comm.make_op(_lib.OP_SENDRECV, _lib.BYTES, world * n, {0: ptrs[0]}, {1: ptrs[1]},
                            [0, 1], route_len=2)
    comm = make_comm(world, spin_budget=1)
    d = describe(comm)
    assert d.origin_cus > 0
    comm.launch(d)
    with pytest.raises(RingTimeout):
        comm.check()
    comm.spin_budget = 400000
    for r in range(world):
        bufs[r].copy_(host[r])
    comm.launch(describe(comm))
    comm.check()
    if op == "broadcast":
        assert all(torch.equal(b.cpu(), host[0]) for b in bufs)
    elif op == "allgather":
        want = torch.stack([host[r][r] for r in range(world)])
        assert all(torch.equal(b.cpu(), want) for b in bufs)
    else:
        assert torch.equal(bufs[1].cpu(), host[0])


def test_residency_is_checked(dev):
    from mintccl_amd import _lib
    world = 8
    comm = make_comm(world, buff_size_=64 << 20, nslots=8, waves_per_rank=8192)
    bufs = [torch.zeros(world, 4096, dtype=torch.float16, device=dev) for _ in range(world)]
    from mintccl_amd.reducescatter import reducescatter
    with pytest.raises(_lib.MintError) as e:
        comm.run(lambda r: reducescatter(bufs[r], comm))
    assert e.value.code == _lib.ERR_RESIDENCY


def test_residency_limit_is_where_the_grid_stops_fitting(dev):
    """6 blocks of 4 waves per CU are accepted, the 7th that the occupancy query
    would allow is not: such grids were measured to run in more than one go."""
    from mintccl_amd import _lib
    from mintccl_amd.reducescatter import reducescatter
    world = 8
    bufs = [torch.zeros(world, 4096, dtype=torch.float16, device=dev) for _ in range(world)]
    cu = torch.cuda.get_device_properties(dev).multi_processor_count
    # blocks = 8 pipelines x 9 positions x (waves / 4): 84 waves -> 1512 blocks, 88 -> 1584
    ok = make_comm(world, buff_size_=2 * 84 * 8 * 1024, nslots=2, waves_per_rank=84 * 8)
    ok.run(lambda r: reducescatter(bufs[r], ok))
    ok.check()
    assert ok.last_grid == 1512 <= 6 * cu
    over = make_comm(world, buff_size_=2 * 88 * 8 * 1024, nslots=2, waves_per_rank=88 * 8)
    assert 6 * cu < 1584 <= 7 * cu
    with pytest.raises(_lib.MintError) as e:
        over.run(lambda r: reducescatter(bufs[r], over))
    assert e.value.code == _lib.ERR_RESIDENCY


def run_probe(lib, dev, pairs, iters, cp, place, per_sector):
    st = torch.zeros(pairs * (4 * 1024 + 128), dtype=torch.uint8, device=dev)
    cnt = torch.zeros(8, dtype=torch.int64, device=dev)
    assert lib.mint_torn_line_probe(st.data_ptr(), st.numel(), pairs, iters, cp, place, per_sector,
                                    3, 400000, cnt.data_ptr(), 0) == 0
    torch.cuda.synchronize()
    return cnt.cpu().tolist()


@pytest.mark.parametrize("cp,place", [(0, 0), (0, 1), (1, 0), (1, 1), (2, 1)])
def test_no_torn_sectors(lib, dev, cp, place):
    # every 64-byte sector carries its tag and a payload that is a function of
    # the tag: once all 16 tags of a block are seen, every byte must belong
    pairs, iters = 2048, 20000
    checked, torn, polls, timeouts, first_half = run_probe(lib, dev, pairs, iters, cp, place, 1)[:5]
    assert timeouts == 0 and checked == pairs * iters * 8
    assert torn == 0


def test_one_flag_per_128_byte_line_is_not_enough(lib, dev):
    # the reference's assumption (protocol.py:31-35): whoever sees the flag in
    # the last bytes of a 128-byte line has the whole line.  On this GPU the
    # first 64-byte sector can still be the old one; whenever that is
    # observed it is exactly that sector, never a finer tear.
    pairs, iters = 2048, 20000
    checked, torn, polls, timeouts, first_half = run_probe(lib, dev, pairs, iters, 0, 0, 0)[:5]
    assert timeouts == 0 and checked == pairs * iters * 8
    print(f"lines checked {checked}, torn {torn} (first sector stale: {first_half})")
    # How often a line tears depends on the machine's load and may be zero in
    # a short run; what is pinned is the shape of a tear when there is one.
    if torn:
        assert torn == first_half


# ---- the benchmark configurations at their full sizes -----------------------
def test_config3_broadcast_64mib_8_ranks(dev):
    world, n = 8, 33554432
    root_data = uniform(n, -4.0, 4.0, 2).to(dev)
    bufs = [root_data.clone() if r == 0 else torch.zeros(n, dtype=torch.float16, device=dev)
            for r in range(world)]
    comm = make_comm(world, buff_size_=8 * 512 * 1024, nslots=8)
    run_broadcast(comm, bufs, 0)
    for b in bufs:
        assert torch.equal(b.view(torch.int16), root_data.view(torch.int16))


@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
def test_config4_reducescatter_and_reduce_32m_elements(dev, dt):
    # 32 Mi elements per rank, seed 3000 + rank, 1 MiB slots.  Every owner row,
    # whole, against the oracle's fold on the host (the arithmetic and the
    # order at full size); rows a rank does not own must come back untouched.
    # The device adder folded in ring order is kept beside it as a second,
    # independent route to the same bits.
    from mintccl_amd import primitive
    world, n_total = 8, 33554432
    n = n_total // world
    host = [normal(n_total, 3000 + r, TORCH_DT[dt]).reshape(world, n) for r in range(world)]
    bufs = [h.to(dev) for h in host]
    orig = [b.clone() for b in bufs]
    comm = make_comm(world, buff_size_=8 << 20, nslots=8, waves_per_rank=256)
    run_reducescatter(comm, bufs)
    for c in range(world):
        want = ring.fold([as_bytes(host[r][c]) for r in range(world)],
                         ring.fold_order(ring.identity_ring(world), c), dt)
        assert np.array_equal(as_bytes(bufs[c][c]), want), c
        acc = orig[c][c].clone()
        for k in range(1, world):
            acc = primitive.Sum(orig[(c + k) % world][c].contiguous(), acc)
        assert torch.equal(bufs[c][c].view(torch.uint8), acc.view(torch.uint8))
        for r in range(world):
            if r != c:
                assert torch.equal(bufs[r][c], orig[r][c])
    flat = [o.reshape(-1).clone() for o in orig]
    run_reduce(comm, flat, 0)
    want = ring.fold([as_bytes(h) for h in host], ring.fold_order(ring.identity_ring(world), 0), dt)
    assert np.array_equal(as_bytes(flat[0]), want)
    for r in range(1, world):
        assert torch.equal(flat[r], orig[r].reshape(-1))


def test_headline_reducescatter_256mib_fp16(dev):
    """8 ranks x 256 MiB fp16 with the library's default geometry (the one
    bench.py times): every owner row, all 32 MiB of it, against the oracle's
    fold computed on the host, and every other row untouched."""
    from mintccl_amd import primitive
    world, n_total = 8, 134217728
    n = n_total // world
    g = torch.Generator(device=dev).manual_seed(7)
    bufs = [torch.randn(world, n, generator=g, device=dev, dtype=torch.float16) for _ in range(world)]
    orig = [b.clone() for b in bufs]
    comm = make_comm(world)
    run_reducescatter(comm, bufs)
    for c in range(world):
        rows = [as_bytes(orig[r][c]) for r in range(world)]
        want = ring.fold(rows, ring.fold_order(ring.identity_ring(world), c), "f16")
        assert np.array_equal(as_bytes(bufs[c][c]), want), c
        del rows, want
        acc = orig[c][c].clone()
        for k in range(1, world):
            acc = primitive.Sum(orig[(c + k) % world][c].contiguous(), acc)
        assert torch.equal(bufs[c][c].view(torch.int16), acc.view(torch.int16))
        for r in range(world):
            if r != c:
                assert torch.equal(bufs[r][c].view(torch.int16), orig[r][c].view(torch.int16)), (r, c)


def test_empty_buffers_are_a_no_op(dev):
    """Zero bytes: every collective returns without launching and touches nothing."""
    from mintccl_amd.allgather import allgather
    from mintccl_amd.allreduce import allreduce
    from mintccl_amd.broadcast import broadcast
    from mintccl_amd.reduce import reduce
    from mintccl_amd.reducescatter import reducescatter
    world = 4
    comm = make_comm(world)
    rows = [torch.empty(world, 0, dtype=torch.float16, device=dev) for _ in range(world)]
    flat = [torch.empty(0, dtype=torch.float16, device=dev) for _ in range(world)]
    comm.run(lambda r: reducescatter(rows[r], comm))
    comm.run(lambda r: allgather(rows[r], comm))
    comm.run(lambda r: reduce(flat[r], 1, comm))
    comm.run(lambda r: broadcast(flat[r], 2, comm))
    comm.run(lambda r: allreduce(flat[r], comm))
    comm.check()


def test_rows_beyond_4_gib(dev):
    """Offsets inside a row are 64-bit: a 4 GiB + 960 KiB + 40 B message through two
    hops (rank 0 -> 1 -> 2 as a broadcast over 3 ranks) arrives bit for bit."""
    from mintccl_amd.broadcast import broadcast
    n = (4 << 30) + 960 * 1024 + 40
    world = 3
    src = torch.empty(n, dtype=torch.uint8, device=dev)
    # a pattern that differs every 4 GiB: byte i = (i * 2654435761 >> 7) & 255 on 64-bit i
    step = 1 << 28
    for lo in range(0, n, step):
        hi = min(n, lo + step)
        i = torch.arange(lo, hi, dtype=torch.int64, device=dev)
        src[lo:hi] = ((i * 2654435761) >> 7).to(torch.uint8)
        del i
    bufs = [src, torch.zeros(n, dtype=torch.uint8, device=dev), torch.zeros(n, dtype=torch.uint8, device=dev)]
    comm = make_comm(world)
    run_broadcast(comm, bufs, 0)
    for b in bufs[1:]:
        assert torch.equal(b, src)


@pytest.mark.parametrize("proto", [0, 1])
def test_a_smaller_epoch_after_a_larger_one_on_the_same_staging(dev, proto):
    """The epoch of a launch only has to differ from the earlier ones on the
    same staging, not to exceed them: credit words and step counters left by a
    launch with a larger epoch must not pass for this launch's (rows of many
    steps through three slots, so every sender has to wait for credits)."""
    world, n = 8, 200000
    comm = make_comm(world, protocol=proto, buff_size_=3 * 8 * 16 * 1024, nslots=3, waves_per_rank=8 * 16)
    for epoch_before in (900, 40):
        host = rank_rows(world, n, "f16", seed0=5000 + epoch_before)
        bufs = [h.to(dev) for h in host]
        comm.epoch = epoch_before          # the launch takes the next one
        run_reducescatter(comm, bufs)
        assert same(bufs, ring.reducescatter([as_bytes(h) for h in host], "f16"))

