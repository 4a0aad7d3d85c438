"""mint_ring_launch_static - the launch that allocates nothing - against
mint_ring_launch on the same inputs, through the C ABI, bit for bit; and
against the oracle.  Two calls in a row share the library's static scratch
array, the second with a smaller input."""
import ctypes

import numpy as np
import pytest
import torch

from mintccl_amd import _lib
from oracle import ring
from tests.helpers import as_bytes, rank_rows, uniform

WORLD = 8


def descriptor(op, dtype, protocol, row_bytes, ptrs, status, root=0, slot_bytes=8 * 64 * 1024,
               nslots=2, waves=16):
    d = _lib.RingOp()
    d.op, d.protocol, d.dtype, d.world = op, protocol, dtype, WORLD
    for i in range(WORLD + 1):
        d.ring[i] = i % WORLD
    d.root = root
    for r in range(WORLD):
        d.input[r] = d.output[r] = ptrs[r]
    d.count_bytes = row_bytes
    d.row_stride = row_bytes if op in (_lib.OP_REDUCESCATTER, _lib.OP_ALLGATHER) else 0
    d.slot_bytes, d.nslots = slot_bytes, nslots
    d.waves_per_channel_group, d.threads_per_block = waves, 256
    d.placement, d.cache_policy = _lib.PLACE_SPREAD, 0
    d.spin_budget = 400000
    d.status = status.data_ptr()
    return d


def launch_allocated(L, d, dev, epoch):
    """The existing entry point, with staging the caller allocates."""
    d.flag_epoch = epoch
    need = L.mint_ring_staging_bytes(d)
    assert need > 0
    staging = torch.zeros(WORLD * need, dtype=torch.uint8, device=dev)
    for r in range(WORLD):
        d.staging[r] = staging.data_ptr() + r * need
    d.staging_bytes = need
    _lib.check(L.mint_ring_launch(d, None), "mint_ring_launch")
    torch.cuda.synchronize()
    return staging


def launch_static(L, d):
    for r in range(WORLD):
        d.staging[r] = 0            # ignored: the library brings its own
    d.staging_bytes = d.flag_epoch = d.epoch_ptr = d.credit_offset = 0
    _lib.check(L.mint_ring_launch_static(d, None), "mint_ring_launch_static")
    torch.cuda.synchronize()


def ok(status):
    return status.cpu().tolist() == [0, 0, 0, 0]


@pytest.mark.gpu
def test_static_launch_matches_the_allocating_launch_twice_in_a_row(dev, lib):
    status = torch.zeros(4, dtype=torch.int64, device=dev)
    # second call smaller than the first; both ragged (many steps, partial last block)
    for n in (100003, 4099):
        host = rank_rows(WORLD, n, "f16", seed0=n)
        a = [h.to(dev) for h in host]
        b = [h.to(dev) for h in host]
        da = descriptor(_lib.OP_REDUCESCATTER, _lib.F16, _lib.PROTO_LL128, n * 2,
                        [t.data_ptr() for t in a], status)
        keep = launch_allocated(lib, da, dev, epoch=7)
        assert ok(status)
        db = descriptor(_lib.OP_REDUCESCATTER, _lib.F16, _lib.PROTO_LL128, n * 2,
                        [t.data_ptr() for t in b], status)
        launch_static(lib, db)
        assert ok(status)
        want = ring.reducescatter([as_bytes(h) for h in host], "f16")
        for r in range(WORLD):
            assert torch.equal(a[r].view(torch.int16), b[r].view(torch.int16)), (n, r)
            assert np.array_equal(as_bytes(b[r]), want[r]), (n, r)
        del keep


@pytest.mark.gpu
def test_static_launch_ll128_after_simple_and_other_geometries(dev, lib):
    """The array keeps the last call's contents: a Simple broadcast whose payload
    is what the next LL128 launch would take for its sector tags, then LL128
    collectives of other shapes on the same array."""
    status = torch.zeros(4, dtype=torch.int64, device=dev)
    # (the epoch in the array is unknown here - other tests may have used it -
    # so the payload forges the tags of every epoch the next launch could carry)
    forged_simple_broadcast(lib, dev, status)
    assert ok(status)
    for n, slot, nslots, waves in ((52000, 8 * 32 * 1024, 4, 32), (480, 8 * 1024, 1, 1)):
        host = [uniform(WORLD * n, -1.0, 1.0, 40 + r).reshape(WORLD, n) for r in range(WORLD)]
        g = [h.to(dev) for h in host]
        d = descriptor(_lib.OP_ALLGATHER, _lib.BYTES, _lib.PROTO_LL128, n * 2,
                       [t.data_ptr() for t in g], status, slot_bytes=slot, nslots=nslots,
                       waves=waves)
        launch_static(lib, d)
        assert ok(status)
        want = ring.allgather([as_bytes(h) for h in host])
        for r in range(WORLD):
            assert np.array_equal(as_bytes(g[r]), want[r]), (n, r)


@pytest.mark.gpu
def test_static_launch_of_the_tree_and_the_temporal_schedule(dev, lib):
    """The newer walks through the same static array: a reduce up the binary tree
    (two shares per slot) and the allgather that moves row after row."""
    status = torch.zeros(4, dtype=torch.int64, device=dev)
    n = 30011
    host = [uniform(n, -1.0, 1.0, 70 + r) for r in range(WORLD)]
    bufs = [h.to(dev) for h in host]
    d = descriptor(_lib.OP_TREE_REDUCE, _lib.F16, _lib.PROTO_LL128, n * 2,
                   [t.data_ptr() for t in bufs], status, root=5, slot_bytes=2 * 32 * 1024, nslots=3,
                   waves=32)
    launch_static(lib, d)
    assert ok(status)
    want = ring.tree_reduce([as_bytes(h) for h in host], 5, "f16")
    for r in range(WORLD):
        assert np.array_equal(as_bytes(bufs[r]), want[r]), r
    m = 9001
    host = [uniform(WORLD * m, -1.0, 1.0, 80 + r).reshape(WORLD, m) for r in range(WORLD)]
    g = [h.to(dev) for h in host]
    d = descriptor(_lib.OP_ALLGATHER_TEMPORAL, _lib.BYTES, _lib.PROTO_LL128, m * 2,
                   [t.data_ptr() for t in g], status, slot_bytes=8 * 1024, nslots=2, waves=8)
    d.row_stride = m * 2
    launch_static(lib, d)
    assert ok(status)
    want = ring.allgather([as_bytes(h) for h in host])
    for r in range(WORLD):
        assert np.array_equal(as_bytes(g[r]), want[r]), r


@pytest.mark.gpu
def test_static_launch_over_the_hypercube(dev, lib):
    """Recursive halving and doubling through the static array (seven shares
    per slot), under the local placement too."""
    status = torch.zeros(4, dtype=torch.int64, device=dev)
    n = 20011
    for placement, cache in ((_lib.PLACE_SPREAD, 0), (_lib.PLACE_LOCAL, 2)):
        host = rank_rows(WORLD, n, "f16", seed0=90)
        bufs = [h.to(dev) for h in host]
        d = descriptor(_lib.OP_HYPERCUBE_REDUCESCATTER, _lib.F16, _lib.PROTO_LL128, n * 2,
                       [t.data_ptr() for t in bufs], status, slot_bytes=7 * 16 * 1024, nslots=3,
                       waves=16)
        d.row_stride = n * 2
        d.placement, d.cache_policy = placement, cache
        launch_static(lib, d)
        assert ok(status)
        want = ring.hypercube_reducescatter([as_bytes(h) for h in host], "f16")
        for r in range(WORLD):
            assert np.array_equal(as_bytes(bufs[r]), want[r]), r
        d = descriptor(_lib.OP_HYPERCUBE_ALLGATHER, _lib.BYTES, _lib.PROTO_LL128, n * 2,
                       [t.data_ptr() for t in bufs], status, slot_bytes=7 * 16 * 1024, nslots=3,
                       waves=16)
        d.row_stride = n * 2
        d.placement, d.cache_policy = placement, cache
        launch_static(lib, d)
        assert ok(status)
        for r, w in enumerate(ring.allgather(want)):
            assert np.array_equal(as_bytes(bufs[r]), w), r


def forged_simple_broadcast(lib, dev, status):
    """A Simple broadcast through the static array whose payload is what an
    LL128 launch of any epoch would take for its sector tags."""
    n32 = 3 * 5 * 7 * 1024 + 3
    src = torch.arange(n32, dtype=torch.int64)
    forged = ((((src // 256) % 4095 + 1) << 20) | 1).to(torch.int32)
    bufs = [forged.to(dev) if r == 2 else torch.zeros(n32, dtype=torch.int32, device=dev)
            for r in range(WORLD)]
    d = descriptor(_lib.OP_BROADCAST, _lib.BYTES, _lib.PROTO_SIMPLE, n32 * 4,
                   [t.data_ptr() for t in bufs], status, root=2, slot_bytes=64 * 1024, nslots=3)
    launch_static(lib, d)
    for t in bufs:
        assert torch.equal(t.cpu(), forged)


@pytest.mark.gpu
def test_static_launch_captured_then_replayed_after_a_simple_launch(dev, lib):
    """An LL128 launch through the static array is captured into a graph while
    the launch before it was LL128 as well.  Between the replays an eager
    Simple launch leaves payload in the array that would pass for sector tags:
    every replay has to clear it by itself (the decision is taken on the
    device when the graph runs, not on the host when it was captured) and
    equal the oracle."""
    status = torch.zeros(4, dtype=torch.int64, device=dev)
    assert lib.mint_static_init() == _lib.OK
    n = 52000
    ins = [torch.zeros(WORLD, n, dtype=torch.float16, device=dev) for _ in range(WORLD)]
    g = [torch.zeros_like(x) for x in ins]
    d = descriptor(_lib.OP_ALLGATHER, _lib.BYTES, _lib.PROTO_LL128, n * 2,
                   [t.data_ptr() for t in g], status, slot_bytes=8 * 32 * 1024, nslots=4, waves=32)
    for r in range(WORLD):
        d.staging[r] = 0
    d.staging_bytes = d.flag_epoch = d.epoch_ptr = d.credit_offset = 0
    side = torch.cuda.Stream(device=dev)

    def enqueue():
        for r in range(WORLD):
            g[r].copy_(ins[r])
        _lib.check(lib.mint_ring_launch_static(d, side.cuda_stream), "mint_ring_launch_static")

    with torch.cuda.stream(side):
        enqueue()                                  # LL128 before the capture
    side.synchronize()
    assert ok(status)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        enqueue()
    for replay in range(4):
        host = [uniform(WORLD * n, -1.0, 1.0, 900 + 10 * replay + r).reshape(WORLD, n)
                for r in range(WORLD)]
        for r in range(WORLD):
            ins[r].copy_(host[r].to(dev))
        if replay % 2 == 0:
            forged_simple_broadcast(lib, dev, status)   # eager, between the replays
            assert ok(status)
        graph.replay()
        torch.cuda.synchronize()
        assert ok(status), replay
        want = ring.allgather([as_bytes(h) for h in host])
        for r in range(WORLD):
            assert np.array_equal(as_bytes(g[r]), want[r]), (replay, r)


@pytest.mark.gpu
def test_static_launch_allocates_nothing_and_queues_back_to_back(dev, lib):
    """A warm call leaves the device's free memory as it was, and two launches
    queued on one stream with no host synchronisation in between (they share
    the array, the stream orders them) both equal the oracle."""
    status = torch.zeros(4, dtype=torch.int64, device=dev)
    n = 30011
    hosts, bufs, descs = [], [], []
    for k in range(2):
        host = rank_rows(WORLD, n - 1000 * k, "f16", seed0=500 + 20 * k)
        b = [h.to(dev) for h in host]
        d = descriptor(_lib.OP_REDUCESCATTER, _lib.F16, _lib.PROTO_LL128, (n - 1000 * k) * 2,
                       [t.data_ptr() for t in b], status)
        for r in range(WORLD):
            d.staging[r] = 0
        d.staging_bytes = d.flag_epoch = d.epoch_ptr = d.credit_offset = 0
        hosts.append(host); bufs.append(b); descs.append(d)
    warm = [h.to(dev) for h in hosts[0]]
    dw = descriptor(_lib.OP_REDUCESCATTER, _lib.F16, _lib.PROTO_LL128, n * 2,
                    [t.data_ptr() for t in warm], status)
    launch_static(lib, dw)
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info(dev)
    reserved_before = torch.cuda.memory_reserved(dev)
    for d in descs:
        _lib.check(lib.mint_ring_launch_static(d, None), "mint_ring_launch_static")
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info(dev)
    assert free_after == free_before and torch.cuda.memory_reserved(dev) == reserved_before
    assert ok(status)
    for host, b in zip(hosts, bufs):
        want = ring.reducescatter([as_bytes(h) for h in host], "f16")
        for r in range(WORLD):
            assert np.array_equal(as_bytes(b[r]), want[r]), r


def test_static_launch_refuses_what_does_not_fit_the_array():
    """Size limits are checked before any device is touched."""
    L = _lib.lib()
    status = ctypes.c_uint64 * 4
    d = _lib.RingOp()
    d.op, d.protocol, d.dtype, d.world = _lib.OP_REDUCESCATTER, _lib.PROTO_LL128, _lib.F16, WORLD
    for i in range(WORLD + 1):
        d.ring[i] = i % WORLD
    for r in range(WORLD):
        d.input[r] = d.output[r] = 0x10000000 + r * 0x1000000
    d.count_bytes = d.row_stride = 1 << 20
    d.threads_per_block, d.status = 256, 0x60000000
    # slots beyond MINT_STATIC_SLOT_BYTES
    d.slot_bytes, d.nslots, d.waves_per_channel_group = 512 << 10, 4, 16
    assert L.mint_ring_launch_static(d, None) == _lib.ERR_TOO_LARGE
    # more wave-channels per rank than there are credit lines (8 pipelines x 144 > 1024)
    d.slot_bytes, d.nslots, d.waves_per_channel_group = 8 * 144 * 1024, 1, 144
    assert L.mint_ring_launch_static(d, None) == _lib.ERR_TOO_LARGE
    # other descriptor errors are reported as by mint_ring_launch
    d.slot_bytes, d.nslots, d.waves_per_channel_group = 512 << 10, 2, 7
    assert L.mint_ring_launch_static(d, None) == _lib.ERR_GEOMETRY
    assert L.mint_ring_launch_static(None, None) == _lib.ERR_ARG
    del status
