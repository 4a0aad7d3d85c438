"""Seats under the local placement (``MINT_PLACE_LOCAL``): which (pipeline,
position, thread block of the position's group) a block takes, listed on the
host by the code the kernels run (``mint_ring_seat``).  No GPU needed.

A block claims an entry of the list of the XCD it finds itself on through
counters: the compute unit that was the j-th of its XCD to show up takes, with
its n-th block, entry n * 32 + j; what is left goes by leftover ticket.  The
reference has nothing of the kind (``7_reducescatter.py:23-25`` maps
``program_id`` to its work directly: every rank is a GPU of its own).  What
has to hold: whatever order the device deals its blocks in - over the XCDs,
over the compute units of an XCD, and whatever order they reach the counters
in - every seat is taken exactly once, as long as every XCD receives an
eighth of the grid and every compute unit its share of that; and when a
compute unit falls short, a seat stays empty (which the kernels detect before
anything is stored into a caller's buffer)."""
import ctypes
import random

import pytest

from mintccl_amd import _lib
from tests.test_abi import make_op

XCDS, CUS = 8, 32


def op_for(**kw):
    d = make_op(**kw)
    d.row_stride = d.count_bytes            # rows of allgather / reducescatter: back to back
    if d.op == _lib.OP_SENDRECV:
        d.route_len = 2
    return d


def seats_for(d, deal):
    """Simulate a launch: `deal(xcd, count)` returns, for the `count` blocks an
    XCD receives, the hardware compute unit of each in the order in which they
    reach the counters.  Returns the list of seats taken."""
    L = _lib.lib()
    grid = L.mint_ring_grid_blocks(d)
    assert grid > 0 and grid % XCDS == 0
    taken = []
    for xcd in range(XCDS):
        rank_of, arrived, leftover = {}, {}, 0
        for cu in deal(xcd, grid // XCDS):
            j = rank_of.setdefault(cu, len(rank_of))
            n = arrived.get(cu, 0)
            arrived[cu] = n + 1
            used, p, h, b = (ctypes.c_int(0) for _ in range(4))
            rc = L.mint_ring_seat(d, xcd, j, n, leftover, ctypes.byref(used), ctypes.byref(p),
                                  ctypes.byref(h), ctypes.byref(b))
            assert rc in (0, 1), rc
            leftover += used.value
            if rc == 1:
                taken.append((p.value, h.value, b.value))
    return taken


def all_seats(d):
    pipes = {_lib.OP_ALLGATHER: d.world, _lib.OP_REDUCESCATTER: d.world, _lib.OP_ALLREDUCE: d.world,
             _lib.OP_ALLTOALL: d.world * d.world, _lib.OP_HYPERCUBE_REDUCESCATTER: d.world,
             _lib.OP_HYPERCUBE_ALLGATHER: d.world}.get(d.op, 1)
    npos = {_lib.OP_SENDRECV: d.route_len, _lib.OP_BROADCAST: d.world, _lib.OP_ALLGATHER: d.world,
            _lib.OP_ALLGATHER_TEMPORAL: d.world, _lib.OP_TREE_BROADCAST: d.world,
            _lib.OP_TREE_REDUCE: d.world, _lib.OP_ALLREDUCE: 2 * d.world - 1,
            _lib.OP_ALLTOALL: 2, _lib.OP_HYPERCUBE_REDUCESCATTER: d.world,
            _lib.OP_HYPERCUBE_ALLGATHER: d.world}.get(d.op, d.world + 1)
    threads = min(d.threads_per_block, d.waves_per_channel_group * 64)
    groups = -(-d.waves_per_channel_group * 64 // threads)
    return {(p, h, b) for p in range(pipes) for h in range(npos) for b in range(groups)}


def in_turn(order):
    """The compute units of an XCD take blocks in turn, in `order`."""
    return lambda xcd, count: [order[i % CUS] for i in range(count)]


def shuffled(seed):
    """Every compute unit gets its share, but the blocks reach the counters in
    any order (as they do: a block's first instructions take longer than the
    dispatch of the next thirty)."""
    def deal(xcd, count):
        cus = [(i % CUS) * 7 % 251 for i in range(count)]          # sparse hardware numbers
        random.Random(seed * 8 + xcd).shuffle(cus)
        return cus
    return deal


LOCAL = dict(placement=_lib.PLACE_LOCAL, cache_policy=2)
CASES = [
    # the headline launch: 8 x 9 positions x 28 blocks of two wave-channels (2016 blocks: 7.875 rounds)
    dict(op=_lib.OP_REDUCESCATTER, count_bytes=32 << 20, slot_bytes=448 << 10, nslots=3,
         waves_per_channel_group=56, threads_per_block=128, **LOCAL),
    # allgather with compute units set apart for the origins (whole rounds, empty entries)
    dict(op=_lib.OP_ALLGATHER, dtype=_lib.BYTES, count_bytes=128 << 20, slot_bytes=512 << 10, nslots=3,
         waves_per_channel_group=64, threads_per_block=256, origin_cus=9, **LOCAL),
    dict(op=_lib.OP_BROADCAST, dtype=_lib.BYTES, count_bytes=64 << 20, slot_bytes=512 << 10, nslots=3,
         waves_per_channel_group=512, threads_per_block=256, origin_cus=9, root=3, **LOCAL),
    # positions turned from round to round (tree, temporal)
    dict(op=_lib.OP_TREE_REDUCE, count_bytes=64 << 20, slot_bytes=2 * 512 << 10, nslots=3,
         waves_per_channel_group=512, threads_per_block=256, root=5, **LOCAL),
    dict(op=_lib.OP_ALLGATHER_TEMPORAL, dtype=_lib.BYTES, count_bytes=8 << 20, slot_bytes=512 << 10,
         nslots=3, waves_per_channel_group=512, threads_per_block=256, origin_cus=9, **LOCAL),
    # small grids: less than one round, and a list that is no multiple of 32
    dict(op=_lib.OP_ALLGATHER, dtype=_lib.BYTES, count_bytes=4096, slot_bytes=8 << 10, nslots=3,
         waves_per_channel_group=1, threads_per_block=64, **LOCAL),
    dict(op=_lib.OP_REDUCE, count_bytes=1 << 20, slot_bytes=40 << 10, nslots=2,
         waves_per_channel_group=40, threads_per_block=64, root=1, **LOCAL),
    dict(op=_lib.OP_ALLREDUCE, count_bytes=16 << 20, slot_bytes=16 * 24 << 10, nslots=3,
         waves_per_channel_group=24, threads_per_block=192, **LOCAL),
    # a hypercube: 8 rows x 8 corners
    dict(op=_lib.OP_HYPERCUBE_REDUCESCATTER, count_bytes=8 << 20, slot_bytes=7 * 72 << 10, nslots=3,
         waves_per_channel_group=72, threads_per_block=256, **LOCAL),
]


@pytest.mark.parametrize("kw", CASES)
def test_every_seat_exactly_once_whatever_the_order_of_arrival(kw):
    d = op_for(**kw)
    want = all_seats(d)
    deals = [in_turn(list(range(CUS))), in_turn(list(range(CUS))[::-1]),
             in_turn([c * 8 % 251 for c in range(CUS)])] + [shuffled(s) for s in range(4)]
    for deal in deals:
        taken = seats_for(d, deal)
        assert len(taken) == len(set(taken)), "a seat was taken twice"
        assert set(taken) == want


def uneven(xcd_short):
    """One compute unit of one XCD gets two blocks fewer than its share and
    its neighbour two more."""
    def deal(xcd, count):
        cus = [i % CUS for i in range(count)]
        if xcd == xcd_short:
            moved = 0
            for i, c in enumerate(cus):
                if c == 5 and moved < 2:
                    cus[i] = 6
                    moved += 1
        return cus
    return deal


def test_a_compute_unit_that_falls_short_leaves_seats_empty():
    # a tree reduce: 8 positions, 128 entries per XCD = 4 rounds over the compute
    # units.  The compute unit that gets two blocks too few leaves two entries
    # unclaimed (the kernels then report status 3 before any caller buffer is
    # written); nothing is taken twice
    d = op_for(**CASES[3])
    taken = seats_for(d, uneven(3))
    assert len(taken) == len(set(taken))
    assert len(set(taken)) == len(all_seats(d)) - 2


def test_a_small_launch_is_seated_in_the_order_of_arrival():
    # at most one round (32 entries per XCD): one counter per XCD hands out the
    # entries, so only the XCDs' shares have to be right
    d = op_for(**CASES[5])
    taken = seats_for(d, uneven(3))
    assert len(taken) == len(set(taken)) and set(taken) == all_seats(d)


def test_seat_arguments_are_checked():
    L = _lib.lib()
    d = op_for(**CASES[0])
    none = [None] * 5
    assert L.mint_ring_seat(d, 8, 0, 0, 0, *none) == _lib.ERR_ARG
    assert L.mint_ring_seat(d, 0, -1, 0, 0, *none) == _lib.ERR_ARG
    spread = op_for(**{**CASES[0], "placement": _lib.PLACE_SPREAD, "cache_policy": 0})
    assert L.mint_ring_seat(spread, 0, 0, 0, 0, *none) == _lib.ERR_ARG
    # beyond a compute unit's share and beyond the leftover entries: nothing to do
    assert L.mint_ring_seat(d, 0, 0, 1000, 1000, *none) == 0
