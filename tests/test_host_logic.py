"""Host-side logic that needs no GPU: knobs and wave-count selection."""
import pytest

from mintccl_amd import _lib, common, protocol


def test_reference_constants():
    assert common.NULL == 0 and common.VECTORIZED_BYTES == 16 and common.WARP_SIZE == 64
    assert protocol.BYTES_LL128_MSG == 128 and protocol.BYTES_LL128_RAW == 120
    assert protocol.WORKGROUP_SIZE == 8 and protocol.PAYLOAD_FLAG_THREAD == 8
    assert protocol.BYTES_BLOCK_MSG == 1024 and protocol.BYTES_BLOCK_RAW == 960


def test_env_knobs_are_read_at_call_time(monkeypatch):
    assert common.num_blocks() == 16 and common.num_warps() == 16
    assert common.buff_size() == 4194304 and common.test_count() == 67108864
    monkeypatch.setenv("MINTCCL_NUM_BLOCKS", "32")
    monkeypatch.setenv("MINTCCL_BUFFSIZE", "8388608")
    monkeypatch.setenv("MINTCCL_TEST_MODE", "0")      # any non-empty string (common.py:113)
    assert common.num_blocks() == 32 and common.buff_size() == 8388608
    assert common.test_mode() is True
    monkeypatch.setenv("MINTCCL_PROTOCOL", "simple")
    assert common.protocol_env() == 1


@pytest.mark.parametrize("n,cap,want", [(64, 16, 16), (64, 100, 64), (60, 16, 15), (7, 4, 1),
                                        (512, 128, 128), (1, 5, 1)])
def test_largest_divisor(n, cap, want):
    assert common._largest_divisor_at_most(n, cap) == want


@pytest.mark.parametrize("world", [2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("row_blocks", [None, 1, 37, 5000])
@pytest.mark.parametrize("op", [_lib.OP_SENDRECV, _lib.OP_BROADCAST, _lib.OP_REDUCE, _lib.OP_ALLGATHER,
                                _lib.OP_REDUCESCATTER, _lib.OP_ALLREDUCE, _lib.OP_ALLTOALL,
                                _lib.OP_TREE_BROADCAST, _lib.OP_TREE_REDUCE,
                                _lib.OP_ALLGATHER_TEMPORAL])
def test_tuned_geometry_is_always_launchable(op, world, row_blocks):
    """Whatever the collective and the world size, the tuned geometry passes the
    library's own plan check, deals whole channels to the 8 XCDs, fits its
    staging budget and stays inside the wavefront budget."""
    from tests.test_abi import make_op
    reducing = op in (_lib.OP_REDUCE, _lib.OP_REDUCESCATTER, _lib.OP_ALLREDUCE, _lib.OP_TREE_REDUCE)
    pairs = op in (_lib.OP_REDUCE, _lib.OP_REDUCESCATTER, _lib.OP_ALLREDUCE, _lib.OP_SENDRECV,
                   _lib.OP_ALLTOALL)
    threads = common.TUNED_THREADS_REDUCING if pairs else 256
    slot, nslots, waves = common.tuned_geometry(op, world, 2, threads, common.TUNED_NSLOTS,
                                                row_blocks=row_blocks)
    assert slot % 1024 == 0 and slot <= common.TUNED_SLOT_BUDGET and nslots >= 1
    # (staging is allocated for TUNED_NSLOTS slots of TUNED_SLOT_BUDGET)
    assert nslots * slot <= common.TUNED_NSLOTS * common.TUNED_SLOT_BUDGET
    multi = op == _lib.OP_ALLTOALL
    d = make_op(op=op, world=world, slot_bytes=slot, nslots=nslots, waves_per_channel_group=waves,
                placement=_lib.PLACE_LOCAL, cache_policy=2, route_len=2, threads_per_block=threads,
                dtype=_lib.F16 if reducing else _lib.BYTES)
    pipes = world if op in (_lib.OP_ALLGATHER, _lib.OP_REDUCESCATTER, _lib.OP_ALLREDUCE) else 1
    if op == _lib.OP_ALLTOALL:
        pipes = world * world
    d.origin_cus = common.tuned_origin_cus(op, 2 if op in (_lib.OP_SENDRECV, _lib.OP_ALLTOALL) else world,
                                           pipes * -(-waves // (threads // 64)), threads // 64)
    if op == _lib.OP_ALLTOALL:
        for r in range(8):
            d.output[r] = 0x40000000 + r * 0x1000000
    for i in range(9):
        d.ring[i] = i % world if i < world else 0
    d.ring[world] = 0
    if op == _lib.OP_SENDRECV:
        d.ring[0], d.ring[1] = 0, 1
    if op == _lib.OP_ALLREDUCE:
        d.row_stride = 0
    blocks = _lib.lib().mint_ring_grid_blocks(d)
    assert blocks > 0, blocks
    assert blocks % 8 == 0
    # (CUs set apart for origins fill the grid up to whole rounds over the 256
    # CUs, at most 24 wavefronts each)
    budget = common.TUNED_TOTAL_WAVES_ALLTOALL_SIMPLE if multi else common.TUNED_TOTAL_WAVES
    assert blocks * (threads // 64) <= (24 * 256 if d.origin_cus else budget)
    d.origin_cus = 0
    assert 0 < _lib.lib().mint_ring_grid_blocks(d) <= blocks
    assert _lib.lib().mint_ring_grid_blocks(d) * (threads // 64) <= budget


def test_headline_geometry():
    assert common.tuned_geometry(_lib.OP_REDUCESCATTER, 8, 0, 128, 3) == (448 * 1024, 3, 56)
    assert common.tuned_geometry(_lib.OP_ALLREDUCE, 8, 0, 128, 3) == (512 * 1024, 3, 32)
    assert common.tuned_geometry(_lib.OP_ALLGATHER, 8, 0, 256, 3) == (512 * 1024, 3, 64)
    assert common.tuned_geometry(_lib.OP_BROADCAST, 8, 0, 256, 3) == (512 * 1024, 3, 512)
    assert common.tuned_geometry(_lib.OP_SENDRECV, 8, 2, 128, 3) == (1536 * 1024, 4, 1536)
    assert common.tuned_geometry(_lib.OP_SENDRECV, 8, 3, 128, 3) == (1536 * 1024, 3, 1536)
    assert common.tuned_geometry(_lib.OP_SENDRECV, 8, 2, 128, 3, ll128=False) == (2304 * 1024, 3, 2304)
    assert common.tuned_origin_cus(_lib.OP_SENDRECV, 2, 768, 2) == 20
    assert common.tuned_origin_cus(_lib.OP_ALLGATHER, 8, 8 * 16, 4) == 9
    assert common.tuned_origin_cus(_lib.OP_BROADCAST, 8, 128, 4) == 9
    assert common.tuned_origin_cus(_lib.OP_REDUCESCATTER, 8, 128, 4) == 0
    assert common.tuned_geometry(_lib.OP_ALLTOALL, 8, 0, 128, 3) == (8 * 20 * 1024, 6, 20)
    assert common.tuned_geometry(_lib.OP_ALLTOALL, 8, 0, 128, 3, ll128=False) == (8 * 44 * 1024, 2, 44)
    assert common.tuned_origin_cus(_lib.OP_ALLTOALL, 2, 64 * 10, 2) == 20
    # a small message takes a small grid: the wave-channels are capped at the
    # blocks of one row, in whole thread blocks that the 8 XCDs divide
    assert common.tuned_geometry(_lib.OP_ALLGATHER, 8, 0, 256, 3, row_blocks=1) == (32 * 1024, 3, 4)
    assert common.tuned_geometry(_lib.OP_ALLGATHER, 8, 0, 256, 3, row_blocks=61) == (512 * 1024, 3, 64)
    assert common.tuned_geometry(_lib.OP_ALLGATHER, 8, 0, 256, 3, row_blocks=53) == (448 * 1024, 3, 56)
    assert common.tuned_geometry(_lib.OP_ALLGATHER, 8, 0, 256, 3, row_blocks=10 ** 6) == (512 * 1024, 3, 64)
    assert common.tuned_geometry(_lib.OP_BROADCAST, 8, 0, 256, 3, row_blocks=5) == (32 * 1024, 3, 32)
    assert common.tuned_geometry(_lib.OP_TREE_REDUCE, 8, 0, 256, 3, row_blocks=5) == (2 * 32 * 1024, 3, 32)
    assert common.tuned_geometry(_lib.OP_TREE_REDUCE, 8, 0, 256, 3) == (2 * 512 * 1024, 3, 512)
