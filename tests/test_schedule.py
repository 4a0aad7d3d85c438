"""Properties of the chunk scheduler (which blocks of a row a wave-channel
moves, and where they sit in staging), listed on the host by the same code the
kernels walk (``mint_ring_schedule``).  No GPU needed.

The reference states the mapping inline in its kernels (for the spatial
split e.g. ``7_reducescatter.py:23-34,43-44,75-77``); what it must satisfy is
independent of either formulation: over the wave-channels of one (pipeline,
position) every block of the row is handled exactly once, a step's blocks sit
in distinct 1 KiB cells of the step's slot, slots rotate with the step, and
the cells a sender writes are the cells the next position reads."""
import ctypes

import numpy as np
import pytest

from mintccl_amd import _lib
from tests.test_abi import make_op


def schedule(d, pipeline, position, wave):
    L = _lib.lib()
    n = ctypes.c_uint32(0)
    assert L.mint_ring_schedule(d, pipeline, position, wave, 0, None, None, None, None,
                                ctypes.byref(n)) == _lib.OK
    arrs = [(ctypes.c_uint32 * max(1, n.value))() for _ in range(4)]
    assert L.mint_ring_schedule(d, pipeline, position, wave, n.value, *arrs,
                                ctypes.byref(n)) == _lib.OK
    return [np.ctypeslib.as_array(a)[: n.value].astype(np.int64) for a in arrs]


CASES = [
    # op, protocol, count_bytes per row, slot_bytes, nslots, waves: unroll 1, 2, 4; ragged ends
    dict(op=_lib.OP_REDUCESCATTER, count_bytes=1 << 20, slot_bytes=512 << 10, waves_per_channel_group=64),
    dict(op=_lib.OP_REDUCESCATTER, count_bytes=(1 << 20) + 16, slot_bytes=512 << 10,
         waves_per_channel_group=32),                      # 2 blocks per wave and step
    dict(op=_lib.OP_REDUCESCATTER, count_bytes=(3 << 20) + 4000 * 16, slot_bytes=512 << 10,
         waves_per_channel_group=16, nslots=3),            # 4 per wave and step
    dict(op=_lib.OP_REDUCESCATTER, count_bytes=960 * 7 + 16, slot_bytes=24 << 10, nslots=2,
         waves_per_channel_group=1),                       # 3 per wave and step: unroll 1, 3 groups
    dict(op=_lib.OP_ALLGATHER, dtype=_lib.BYTES, protocol=_lib.PROTO_SIMPLE, count_bytes=(1 << 20) + 48,
         slot_bytes=256 << 10, waves_per_channel_group=8),
    dict(op=_lib.OP_BROADCAST, dtype=_lib.BYTES, count_bytes=5 << 20, slot_bytes=1 << 20, nslots=2,
         waves_per_channel_group=256, root=5),
]


@pytest.mark.parametrize("kw", CASES)
def test_every_block_once_and_cells_distinct(kw):
    d = make_op(**kw)
    if "row_stride" not in kw:
        d.row_stride = (d.count_bytes + 15) // 16 * 16
    assert _lib.lib().mint_ring_grid_blocks(d) > 0
    raw = 960 if d.protocol == _lib.PROTO_LL128 else 1024
    nblocks = -(-d.count_bytes // raw)
    pipes = d.world if d.op in (_lib.OP_ALLGATHER, _lib.OP_REDUCESCATTER) else 1
    share = d.slot_bytes // 1024 // pipes * 1024
    W = d.waves_per_channel_group
    for pipeline in {0, pipes - 1}:
        seen = np.zeros(nblocks, dtype=np.int64)
        cells = {}
        for w in range(W):
            step, block, recv, send = schedule(d, pipeline, 1, w)
            np.add.at(seen, block, 1)
            # a wave-channel's blocks come in ascending order, steps never go back
            assert np.all(np.diff(block) > 0) and np.all(np.diff(step) >= 0)
            # every block in the slot of its step, inside this pipeline's share of it
            slot = recv // d.slot_bytes
            assert np.array_equal(slot, step % d.nslots)
            inside = recv % d.slot_bytes
            assert np.all(inside // share == pipeline) and np.all(recv % 1024 == 0)
            # what position 1 sends is what position 2 receives
            if d.op != _lib.OP_ALLREDUCE:
                _, block2, recv2, _ = schedule(d, pipeline, 2, w)
                assert np.array_equal(block2, block) and np.array_equal(recv2, send)
            for s, c in zip(step.tolist(), recv.tolist()):
                assert (s, c) not in cells
                cells[(s, c)] = w
        assert np.all(seen == 1)


def test_allreduce_phases_have_their_own_cells():
    d = make_op(op=_lib.OP_ALLREDUCE, waves_per_channel_group=16, count_bytes=(8 << 20) + 64)
    d.row_stride = 0
    assert _lib.lib().mint_ring_grid_blocks(d) > 0
    # position 3 adds (phase 0), position 11 = 3 + 8 copies (phase 1): same rank, same blocks
    for w in (0, 15):
        s0, b0, r0, _ = schedule(d, 2, 3, w)
        s1, b1, r1, _ = schedule(d, 2, 11, w)
        assert np.array_equal(b0, b1) and np.array_equal(s0, s1)
        assert not set(r0.tolist()) & set(r1.tolist())
        # the last adder (position 7) sends into phase 1 of the next rank
        _, _, _, send7 = schedule(d, 2, 7, w)
        _, _, recv8, _ = schedule(d, 2, 8, w)
        assert np.array_equal(send7, recv8)
    # the buffer is cut into 8 rows of whole 16-byte vectors; the last row is short
    total = d.count_bytes
    row = (-(-total // 8) + 15) // 16 * 16
    for p in range(8):
        left = max(0, min(row, total - p * row))
        got = sum(len(schedule(d, p, 1, w)[1]) for w in range(16))
        assert got == -(-left // 960)


def test_schedule_rejects_positions_outside_the_launch():
    d = make_op()
    n = ctypes.c_uint32(0)
    L = _lib.lib()
    for args in ((8, 0, 0), (0, 9, 0), (0, 0, 64), (-1, 0, 0)):
        assert L.mint_ring_schedule(d, *args, 0, None, None, None, None, ctypes.byref(n)) == _lib.ERR_ARG
    assert L.mint_ring_schedule(d, 0, 0, 0, 0, None, None, None, None, None) == _lib.ERR_ARG


def test_rows_clipped_to_one_buffer():
    """total_bytes: the rows of a reducescatter / allgather are the pieces of one
    buffer, the last ones short or empty (how an allreduce runs as two launches)."""
    row = 64 * 1024 + 16
    total = 5 * row + 1000 * 2            # rows 0..4 full, row 5 has 2000 bytes, rows 6, 7 empty
    d = make_op(count_bytes=row, row_stride=row, total_bytes=total, waves_per_channel_group=16)
    assert _lib.lib().mint_ring_grid_blocks(d) > 0
    for p, left in enumerate([row] * 5 + [2000, 0, 0]):
        blocks = np.concatenate([schedule(d, p, 1, w)[1] for w in range(16)])
        assert sorted(blocks.tolist()) == list(range(-(-left // 960)))


def test_alltoall_shares_are_per_source_rank():
    """Alltoall: pipeline s * world + d; rank d's slots have one share per
    source rank, so what the origin of (s, d) sends lands in share s of d's
    slot - for every s a different part - and every block goes once."""
    d = make_op(op=_lib.OP_ALLTOALL, dtype=_lib.BYTES, count_bytes=(1 << 20) + 16,
                waves_per_channel_group=16)
    for r in range(8):
        d.output[r] = 0x40000000 + r * 0x1000000
    d.row_stride = d.count_bytes
    assert _lib.lib().mint_ring_grid_blocks(d) == 64 * 2 * 4
    nblocks = -(-d.count_bytes // 960)
    share = d.slot_bytes // 1024 // 8 * 1024
    for s, dst in ((0, 0), (3, 5), (7, 2)):
        p = s * 8 + dst
        seen = np.zeros(nblocks, dtype=np.int64)
        for w in range(16):
            step, block, _, send = schedule(d, p, 0, w)
            step1, block1, recv, _ = schedule(d, p, 1, w)
            np.add.at(seen, block, 1)
            assert np.array_equal(block, block1) and np.array_equal(send, recv)
            assert np.all((send % d.slot_bytes) // share == s)
            assert np.array_equal(send // d.slot_bytes, step % d.nslots)
        assert np.all(seen == 1)
    n = ctypes.c_uint32(0)
    assert _lib.lib().mint_ring_schedule(d, 64, 0, 0, 0, None, None, None, None,
                                         ctypes.byref(n)) == _lib.ERR_ARG
