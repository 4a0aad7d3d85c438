"""Seats under the local placement (``MINT_PLACE_LOCAL``): which (pipeline,
position, thread block of the position's group) a block takes, listed on the
host by the code the kernels run (``mint_ring_seat``).  No GPU needed.

A block claims an entry of the list of the XCD it finds itself on through
counters: the compute unit that was the j-th of its XCD to show up wants, with
its n-th block, entry n * 32 + j; a block that wants none, or finds its entry
taken, draws a ticket and takes the first free entry from the ticket's place
in the last, partial round (later tickets: from the head of the list) upwards.  The reference has nothing of the kind
(``7_reducescatter.py:23-25`` maps ``program_id`` to its work directly: every
rank is a GPU of its own).  What has to hold: whatever way the device deals
its blocks - over the compute units of an XCD (all 32, half of them on a
stream with a CU mask, some of them busy with another kernel), and whatever
order they reach the counters in - every seat is taken exactly once, as long
as every XCD receives an eighth of the grid; and with every compute unit at
its share, a compute unit holds the entries of its own column."""
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


def seats_for(d, deal, with_cu=False):
    """Simulate a launch: `deal(xcd, count)` returns, for the `count` blocks an
    XCD receives, the hardware compute unit of each in the order in which they
    reach the counters.  Returns the list of seats taken."""
    L = _lib.lib()
    grid = L.mint_ring_grid_blocks(d)
    assert grid > 0 and grid % XCDS == 0
    taken = []
    for xcd in range(XCDS):
        rank_of, arrived = {}, {}
        state = (ctypes.c_uint64 * _lib.SEAT_STATE_WORDS)()
        for cu in deal(xcd, grid // XCDS):
            j = rank_of.setdefault(cu, len(rank_of))
            n = arrived.get(cu, 0)
            arrived[cu] = n + 1
            p, h, b = (ctypes.c_int(0) for _ in range(3))
            rc = L.mint_ring_seat(d, xcd, j, n, state, ctypes.byref(p), ctypes.byref(h),
                                  ctypes.byref(b))
            assert rc in (0, 1), rc
            if rc == 1:
                taken.append((p.value, h.value, b.value) if not with_cu else
                             (p.value, h.value, b.value, cu))
    return taken


def L_grid(d):
    return _lib.lib().mint_ring_grid_blocks(d)


def seats_for_xcd(d, xcd, cus):
    """One XCD of a simulated launch: (pipeline, position, block, compute unit) per seat."""
    L = _lib.lib()
    rank_of, arrived, out = {}, {}, []
    state = (ctypes.c_uint64 * _lib.SEAT_STATE_WORDS)()
    for cu in cus:
        j = rank_of.setdefault(cu, len(rank_of))
        n = arrived.get(cu, 0)
        arrived[cu] = n + 1
        p, h, b = (ctypes.c_int(0) for _ in range(3))
        rc = L.mint_ring_seat(d, xcd, j, n, state, ctypes.byref(p), ctypes.byref(h), ctypes.byref(b))
        assert rc in (0, 1), rc
        if rc == 1:
            out.append((p.value, h.value, b.value, cu))
    return out


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
    dict(op=_lib.OP_HYPERCUBE_REDUCESCATTER, count_bytes=8 << 20, slot_bytes=7 * 64 << 10, nslots=3,
         waves_per_channel_group=64, threads_per_block=256, **LOCAL),
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


def masked(keep):
    """A stream confined to `keep` of the 32 compute units of every XCD: they
    take the XCD's blocks in turn, and reach the counters in any order."""
    def deal(xcd, count):
        cus = [(i % keep) * 3 + 1 for i in range(count)]
        random.Random(100 + xcd).shuffle(cus)
        return cus
    return deal


def crowded(xcd, count):
    """Another kernel occupies most of eleven compute units: they take one
    block each, the others share the rest, and one takes a third of the grid."""
    cus = list(range(11)) + [11] * (count // 3)
    cus += [12 + i % 20 for i in range(count - len(cus))]
    random.Random(7 + xcd).shuffle(cus)
    return cus


@pytest.mark.parametrize("kw", CASES)
def test_every_seat_exactly_once_however_uneven_the_deal(kw):
    d = op_for(**kw)
    want = all_seats(d)
    for deal in (uneven(3), masked(16), masked(8), masked(24), masked(5), masked(1), crowded):
        taken = seats_for(d, deal)
        assert len(taken) == len(set(taken)), "a seat was taken twice"
        assert set(taken) == want


def test_with_every_compute_unit_at_its_share_a_compute_unit_holds_one_position():
    # 8 positions, 32 compute units: the entries of a compute unit's column all
    # have the same position, whatever order the blocks reach the counters in;
    # with compute units set apart for the origins, those hold origins only and
    # no other holds one (what the copying collectives' speed rests on)
    for origin_cus in (0, 9):
        d = op_for(**{**CASES[1], "origin_cus": origin_cus})
        per_xcd = L_grid(d) // XCDS
        assert per_xcd % CUS == 0           # whole rounds: nothing is dealt by ticket
        for deal in (in_turn(list(range(CUS))), shuffled(1), shuffled(2)):
            by_cu, taken = {}, []
            for xcd in range(XCDS):
                one = seats_for_xcd(d, xcd, deal(xcd, per_xcd))
                for p, h, b, cu in one:
                    by_cu.setdefault((xcd, cu), []).append(h)
                taken += one
            assert len(taken) == len({t[:3] for t in taken})
            for hs in by_cu.values():
                if origin_cus:
                    assert all(h == 0 for h in hs) or all(h != 0 for h in hs), hs
                else:
                    assert len(set(hs)) == 1, hs
            if origin_cus:
                assert sum(all(h == 0 for h in hs) for hs in by_cu.values()) == XCDS * origin_cus


@pytest.mark.parametrize("case,cus,per_cu", [(0, 16, 12), (0, 8, 16), (1, 16, 5), (3, 16, 6),
                                             (8, 16, 5), (0, 32, 6), (0, 21, 9)])
def test_a_partly_resident_grid_fills_whole_channels(case, cus, per_cu):
    """Where not all blocks of a launch are resident at once (a stream confined
    to `cus` compute units that hold `per_cu` thread blocks each), the blocks
    that are there have to complete channels - every position of a (pipeline,
    block of the group) - so that these finish and make room: played per XCD
    with blocks dealt to the compute units in turn as room becomes free."""
    d = op_for(**CASES[case])
    L = _lib.lib()
    per_xcd = L.mint_ring_grid_blocks(d) // XCDS
    npos = max(h for _, h, _ in all_seats(d)) + 1
    for xcd in range(XCDS):
        state = (ctypes.c_uint64 * _lib.SEAT_STATE_WORDS)()
        rank_of, arrived = {}, {}
        room = {c * 2 + 1: per_cu for c in range(cus)}
        members, holder = {}, {}
        pending, turn, seated = per_xcd, 0, 0
        while pending or members:
            progressed = False
            for _ in range(cus):                         # one round of dispatch
                cu = list(room)[turn % cus]
                turn += 1
                if pending and room[cu]:
                    j = rank_of.setdefault(cu, len(rank_of))
                    n = arrived.get(cu, 0)
                    arrived[cu] = n + 1
                    p, h, b = (ctypes.c_int(0) for _ in range(3))
                    rc = L.mint_ring_seat(d, xcd, j, n, state, ctypes.byref(p), ctypes.byref(h),
                                          ctypes.byref(b))
                    assert rc in (0, 1)
                    pending -= 1
                    progressed = True
                    if rc == 1:                         # (an empty entry: the block exits at once)
                        room[cu] -= 1
                        seated += 1
                        members.setdefault((p.value, b.value), set()).add(h.value)
                        holder.setdefault((p.value, b.value), []).append(cu)
            for key in [k for k, hs in members.items() if len(hs) == npos]:
                for cu in holder.pop(key):
                    room[cu] += 1
                del members[key]
                progressed = True
            assert progressed, f"XCD {xcd}: {len(members)} channels wait for blocks that cannot start"
        assert seated == len(all_seats(d)) // XCDS


def test_random_deals_seat_every_block_exactly_once():
    """Any multiset of compute units, in any order: as many blocks as entries
    means every seat is taken exactly once (25 random launches per case, every XCD its own deal, from one
    compute unit taking everything to 60 compute units sharing)."""
    rng = random.Random(2024)
    for kw in (CASES[0], CASES[1], CASES[3], CASES[7]):
        d = op_for(**kw)
        want = all_seats(d)
        per_xcd = L_grid(d) // XCDS

        def deal(xcd, count):
            ncu = rng.choice((1, 2, 3, 7, 16, 31, 32, 33, 40, 60))
            weights = [rng.random() ** 3 + 0.01 for _ in range(ncu)]
            return rng.choices(range(ncu), weights=weights, k=count)
        for _ in range(25):
            taken = seats_for(d, deal)
            assert len(taken) == len(set(taken)) and set(taken) == want
        assert per_xcd == len(want) // XCDS or kw.get("origin_cus")


def test_a_small_launch_is_seated_in_the_order_of_arrival():
    # at most one round (32 entries per XCD): one counter per XCD hands out the
    # entries, so only the XCDs' shares have to be right
    d = op_for(**CASES[5])
    taken = seats_for(d, uneven(3))
    assert len(taken) == len(set(taken)) and set(taken) == all_seats(d)


def test_seat_arguments_are_checked():
    L = _lib.lib()
    d = op_for(**CASES[0])
    none = [None] * 3
    state = (ctypes.c_uint64 * _lib.SEAT_STATE_WORDS)()
    assert L.mint_ring_seat(d, 8, 0, 0, state, *none) == _lib.ERR_ARG
    assert L.mint_ring_seat(d, 0, -1, 0, state, *none) == _lib.ERR_ARG
    assert L.mint_ring_seat(d, 0, 0, 0, None, *none) == _lib.ERR_ARG
    spread = op_for(**{**CASES[0], "placement": _lib.PLACE_SPREAD, "cache_policy": 0})
    assert L.mint_ring_seat(spread, 0, 0, 0, state, *none) == _lib.ERR_ARG
    # one block more than the list has entries: nothing to do
    per_xcd = L.mint_ring_grid_blocks(d) // XCDS
    for i in range(per_xcd):
        assert L.mint_ring_seat(d, 0, i % CUS, i // CUS, state, *none) == 1
    assert L.mint_ring_seat(d, 0, 0, 1000, state, *none) == 0
