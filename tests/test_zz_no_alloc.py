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
    n32 = 3 * 5 * 7 * 1024 + 3
    # the epoch in the array is unknown here (other tests may have used it):
    # forge the tags of every epoch the next launch could carry, in turn
    src = torch.arange(n32, dtype=torch.int64)
    forged = ((((src // 256) % 4095 + 1) << 20) | 1).to(torch.int32)
    bufs = [forged.to(dev) if r == 2 else torch.zeros(n32, dtype=torch.int32, device=dev)
            for r in range(WORLD)]
    d = descriptor(_lib.OP_BROADCAST, _lib.BYTES, _lib.PROTO_SIMPLE, n32 * 4,
                   [t.data_ptr() for t in bufs], status, root=2, slot_bytes=64 * 1024, nslots=3)
    launch_static(lib, d)
    assert ok(status)
    for t in bufs:
        assert torch.equal(t.cpu(), forged)
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
