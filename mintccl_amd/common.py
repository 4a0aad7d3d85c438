"""Configuration and the virtual-rank communicator.

Mirrors the reference's ``common.py``: the tuning knobs keep their
``MINTCCL_*`` names and defaults (``common.py:85-118``) but are read when an
operator runs, not at import.  ``set_gpu`` / ``send_ptr`` / ``recv_ptr``
(``common.py:10-38``) keep their names; with every rank living in one process
on one GPU they reduce to a device choice and a pointer mailbox.
"""
from __future__ import annotations

import contextlib
import math
import os
import threading
import time

import torch

from . import _lib

NULL = 0                       # common.py:71
WARP_SIZE = 64                 # common.py:104 is 32; a CDNA4 wavefront has 64 lanes
VECTORIZED_BYTES = 16          # common.py:105
SPINS_BEFORE_ABORT = 4000000   # common.py:106 (unused there, enforced here)


def _env_int(name: str, default: int) -> int:
    v = os.getenv(name)
    return int(v) if v not in (None, "") else default


def num_blocks() -> int:        # common.py:85
    return _env_int("MINTCCL_NUM_BLOCKS", 16)


def num_warps() -> int:         # common.py:92 (32-lane warps; two make a wavefront)
    return _env_int("MINTCCL_NUM_WARPS", 16)


def buff_size() -> int:         # common.py:101
    return _env_int("MINTCCL_BUFFSIZE", 4194304)


def num_slots() -> int:
    return _env_int("MINTCCL_NSLOTS", 8)


def world_size_env() -> int:
    return _env_int("MINTCCL_WORLD_SIZE", 8)


def protocol_env() -> int:
    return {"ll128": _lib.PROTO_LL128, "simple": _lib.PROTO_SIMPLE}[
        os.getenv("MINTCCL_PROTOCOL", "ll128").lower()]


def cache_policy_env() -> int:
    return {"agent": 0, "system": 1, "xcd": 2}[os.getenv("MINTCCL_CACHE", "agent").lower()]


def placement_env() -> int:
    return {"spread": _lib.PLACE_SPREAD, "local": _lib.PLACE_LOCAL}[
        os.getenv("MINTCCL_PLACEMENT", "spread").lower()]


def row_fetch_env() -> int:
    return {"inline": _lib.FETCH_INLINE, "lds": _lib.FETCH_LDS}[
        os.getenv("MINTCCL_ROW_FETCH", "inline").lower()]


def test_mode() -> bool:        # common.py:113 (any non-empty string enables it)
    return bool(os.getenv("MINTCCL_TEST_MODE", ""))


def test_count() -> int:        # common.py:115
    return _env_int("MINTCCL_TEST_COUNT", 67108864)


def verbose() -> bool:          # common.py:118
    return bool(os.getenv("MINTCCL_TEST_VERBOSE", ""))


DTYPE_CODE = {torch.float16: _lib.F16, torch.bfloat16: _lib.BF16, torch.float32: _lib.F32}


class Timer:
    """CPU / device timer context manager (``common.py:41-67``)."""

    def __init__(self, device: bool = False, rank: int | None = None) -> None:
        self.rank, self.device, self.elapsed = rank, device, 0.0

    def __enter__(self):
        if self.device:
            self.start = torch.cuda.Event(enable_timing=True)
            self.end = torch.cuda.Event(enable_timing=True)
            self.start.record()
        else:
            self.start = time.perf_counter_ns()
        return self

    def __exit__(self, *exc):
        if self.device:
            self.end.record()
            torch.cuda.synchronize()
            self.elapsed = self.start.elapsed_time(self.end) / 1e3
        else:
            self.elapsed = (time.perf_counter_ns() - self.start) / 1e9
        tag = f"rank: {self.rank} " if self.rank is not None else ""
        print(f"# {tag}time: {self.elapsed}s")


# Tuned geometry for MI355X (measured), one 1 KiB block per wave-channel per
# step.  3 slots of 512 KiB and 4608 wavefronts, with these exceptions:
# reducescatter 3 slots of 448 KiB, 56 wave-channels per (row, hop) instead of
# 64 (1.5 - 2 % faster: 4032 wavefronts are at most 16 on a compute unit, and
# the device serves the collectives' access mix a fifth slower with 18), and
# the ring reduce likewise 448 wave-channels per position (-3 %); an LL128 sendrecv over one hop 4 slots of 1.5 MiB;
# alltoall 6 slots and 2560 wavefronts in all under LL128, 2 slots and 5760
# under Simple.  A slot may grow to TUNED_SLOT_BUDGET bytes when there are few
# hops.  Sendrecv, broadcast, allgather and alltoall set compute units apart
# for their origins (tuned_origin_cus).  The reducing collectives, sendrecv and
# alltoall run thread blocks of 2 wave-channels (TUNED_THREADS_REDUCING;
# sendrecv -9 %, alltoall -7 % against blocks of 4; broadcast the same either
# way, allgather 7 % slower) unless the caller names a block size.  Staging is
# allocated for TUNED_NSLOTS slots of TUNED_SLOT_BUDGET either way.
TUNED_TOTAL_WAVES = 4608
TUNED_SLOT_BLOCKS = 512
TUNED_SLOT_BLOCKS_REDUCESCATTER = 448
TUNED_NSLOTS = 3
TUNED_TOTAL_WAVES_ALLTOALL = 2560
TUNED_NSLOTS_ALLTOALL = 6
TUNED_TOTAL_WAVES_ALLTOALL_SIMPLE = 5760
TUNED_NSLOTS_ALLTOALL_SIMPLE = 2
TUNED_SLOT_BUDGET = 2304 * 1024
TUNED_THREADS_REDUCING = 128
TUNED_SENDRECV_SLOT_BLOCKS = 1536
TUNED_SENDRECV_NSLOTS = 4


class RingTimeout(RuntimeError):
    """A bounded wait inside the ring kernel ran out (status word 0 == 1)."""


class PlacementError(RuntimeError):
    """The local placement ran on a device that numbers its XCDs beyond 7
    (status word 0 == 2) or that did not deal an eighth of the thread blocks
    to every XCD (status word 0 == 3)."""


def tuned_geometry(op: int, world: int, route_len: int, threads_per_block: int,
                   max_nslots: int, fetcher_waves: bool = False,
                   row_blocks: int | None = None, ll128: bool = True) -> tuple[int, int, int]:
    """(slot_bytes, nslots, wave-channels per (pipeline, hop)) of the tuned
    geometry for one collective: the wavefront budget spread over the
    (pipeline, hop) groups, one 1 KiB block per wave-channel per step, whole
    thread blocks, and a channel count the 8 XCDs divide.  ``row_blocks``
    (blocks of one row of the message) caps the wave-channels at what the
    message can occupy: a small collective is a small grid (a device time of
    7 us instead of 9 for an 8-rank allgather of up to 64 KiB per rank)."""
    wpb = max(1, threads_per_block // 64)

    def fit(shares: int, nslots: int, waves: int, granule: int) -> tuple[int, int, int]:
        if row_blocks is not None:
            waves = max(granule, min(waves, -(-row_blocks // granule) * granule))
        return shares * waves * 1024, nslots, waves

    if op == _lib.OP_ALLTOALL:
        # world x world pipelines of two positions; a rank's slot has one share
        # per source rank.  Few wave-channels and many small slots, origins on
        # 20 of 32 CUs: 8 x 256 MiB 1.13 -> 0.91 ms (LL128) against 2 slots and
        # 5760 wavefronts with origins and destinations on half of the CUs each.
        # The Simple protocol takes twice as long that way and keeps 2 slots
        # and 5760 wavefronts.
        total = TUNED_TOTAL_WAVES_ALLTOALL if ll128 else TUNED_TOTAL_WAVES_ALLTOALL_SIMPLE
        granule = wpb * (8 // math.gcd(world * world, 8))      # whole channels for every XCD
        waves = max(granule, total // (2 * world * world) // granule * granule)
        if not ll128:
            nslots = min(max_nslots, TUNED_NSLOTS_ALLTOALL_SIMPLE)
        else:
            nslots = TUNED_NSLOTS_ALLTOALL if max_nslots == TUNED_NSLOTS else max_nslots
        return fit(world, nslots, waves, granule)
    if op in (_lib.OP_TREE_BROADCAST, _lib.OP_TREE_REDUCE):
        # one wavefront per (node, wave-channel); a reducing node's slot has a
        # share per child
        shares = 2 if op == _lib.OP_TREE_REDUCE else 1
        granule = wpb * 8
        waves = max(granule, min(TUNED_SLOT_BLOCKS, TUNED_TOTAL_WAVES // world) // granule * granule)
        return fit(shares, max_nslots, waves, granule)
    if op in (_lib.OP_HYPERCUBE_REDUCESCATTER, _lib.OP_HYPERCUBE_ALLGATHER):
        # world rows x world nodes, one wavefront per (row, node, wave-channel);
        # a rank's slot has a share per stream it receives: world - 1.  4096
        # wavefronts are 16 on every compute unit (with 4608 an 8 x 64 MiB
        # allgather takes 10 % longer)
        granule = wpb
        waves = max(granule, min(TUNED_SLOT_BUDGET // 1024 // max(1, world - 1),
                                 4096 // (world * world)) // granule * granule)
        return fit(max(1, world - 1), max_nslots, waves, granule)
    pipes = world if op in (_lib.OP_ALLGATHER, _lib.OP_REDUCESCATTER, _lib.OP_ALLREDUCE) else 1
    real_pipes = pipes
    if op == _lib.OP_ALLREDUCE:
        pipes *= 2                # a slot is shared by (pipeline, phase): two phases
    npos = {_lib.OP_SENDRECV: max(route_len, 1), _lib.OP_BROADCAST: world,
            _lib.OP_ALLGATHER: world, _lib.OP_ALLGATHER_TEMPORAL: world,
            _lib.OP_ALLREDUCE: 2 * world - 1}.get(op, world + 1)
    receivers = max(1, min(npos - 1, world))
    if op == _lib.OP_ALLREDUCE:
        npos = (npos + 1) // 2    # `pipes` already counts both phases
    # slots sized per 8 receiving ranks keep the staging of an XCD's channels
    # (slots x receivers / 8) well inside its 4 MiB of L2
    per8 = (TUNED_SLOT_BLOCKS_REDUCESCATTER if op in (_lib.OP_REDUCESCATTER, _lib.OP_REDUCE)
            else TUNED_SLOT_BLOCKS)
    total = TUNED_TOTAL_WAVES
    if fetcher_waves:
        # every thread block carries one more wavefront (it streams own rows
        # into LDS) and a CU takes whole blocks: 24 wavefronts per CU, 256 CUs
        total = (24 // (wpb + 1)) * 256 * wpb
    nslots = max_nslots
    slot_blocks = min(per8 * max(1, 8 // receivers), total // npos, TUNED_SLOT_BUDGET // 1024)
    if op == _lib.OP_SENDRECV and npos == 2 and max_nslots == TUNED_NSLOTS and ll128:
        # one hop under LL128, its origins on 20 of 32 CUs: four slots of
        # 1.5 MiB in the room of three of 2.25 (-10 % against those; the Simple
        # protocol takes a quarter longer that way and keeps the three)
        slot_blocks, nslots = TUNED_SENDRECV_SLOT_BLOCKS, TUNED_SENDRECV_NSLOTS
    granule = wpb * (8 // math.gcd(real_pipes, 8))
    waves = max(granule, slot_blocks // pipes // granule * granule)
    return fit(pipes, nslots, waves, granule)


def tuned_origin_cus(op: int, npos: int, channels: int, waves_per_block: int) -> int:
    """Of the 32 CUs of an XCD, how many the origins of a sendrecv, a ring
    broadcast, an allgather or an alltoall get to themselves; ``npos`` = positions of a
    pipeline, ``channels`` = thread blocks per position of the launch (the
    library ignores the number for small grids and other collectives).  A CU
    keeps a bounded number of requests in flight (about 15 KB of loads) and a
    load from HBM takes several times longer than usual while the
    collective's stores keep HBM busy, so the origins' natural share
    of the CUs - one position in ``npos`` - delivers too little: measured
    best at 8 positions is 9 of 32 (allgather of 8 x 128 MiB 3.38 -> 2.57 ms,
    broadcast of 64 MiB 0.237 -> 0.171 ms), 2.25 times the natural share,
    which is what other lengths aim for (a sendrecv over one hop: 20 of 32,
    0.131 -> 0.119 ms for 256 MiB; alltoall, whose pipelines are single hops:
    the same 20).  The grid is filled up to whole rounds
    over the CUs and has to stay resident (24 wavefronts per CU): the largest
    count up to the aim that fits."""
    if op not in (_lib.OP_SENDRECV, _lib.OP_BROADCAST, _lib.OP_ALLGATHER, _lib.OP_ALLTOALL,
                  _lib.OP_ALLGATHER_TEMPORAL, _lib.OP_TREE_BROADCAST) or npos < 2 or channels % 8:
        return 0
    groups, rounds_max = channels // 8, 24 // max(1, waves_per_block)
    for n in range(max(1, min(20, round(72 / npos))), 0, -1):
        rounds = max(-(-groups // n), -(-(npos - 1) * groups // (32 - n)))
        if rounds <= rounds_max:
            return n
    return 0


_XCDS: dict[int, int] = {}


def _xcd_count(device: torch.device) -> int:
    """XCDs the device deals thread blocks over (asked once per device)."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    if index not in _XCDS:
        import ctypes
        n = ctypes.c_int(0)
        with torch.cuda.device(index):
            _lib.check(_lib.lib().mint_device_info(None, ctypes.byref(n), None), "mint_device_info")
        _XCDS[index] = n.value
    return _XCDS[index]


def _largest_divisor_at_most(n: int, cap: int) -> int:
    cap = max(1, min(n, cap))
    for d in range(cap, 0, -1):
        if n % d == 0:
            return d
    return 1


class VirtualComm:
    """N virtual ranks on one GPU: stands in for ``MPI.COMM_WORLD``.

    Every rank owns a disjoint region of one staging allocation
    (``nslots`` slots of ``buff_size / nslots`` bytes plus its credit words).
    Ranks enter with ``with comm.rank(r):`` and call the reference-named
    operators; the call that completes the set of participants enqueues ONE
    fused launch that runs all ranks' kernels.
    """

    def __init__(self, world_size: int | None = None, device: str | torch.device = "cuda:0",
                 buff_size_: int | None = None, nslots: int | None = None,
                 protocol: int | None = None, placement: int | None = None,
                 waves_per_rank: int | None = None, threads_per_block: int | None = None,
                 cache_policy: int | None = None, spin_budget: int = 0,
                 device_epoch: bool | None = None, row_fetch: int | None = None,
                 origin_cus: int | None = None) -> None:
        self.world_size = world_size if world_size is not None else world_size_env()
        if not 1 <= self.world_size <= _lib.MAX_RANKS:
            raise ValueError(f"world_size must be 1..{_lib.MAX_RANKS}")
        self.device = torch.device(device)
        # Geometry.  Explicit arguments win, then the reference's MINTCCL_*
        # knobs (common.py:85-101: NUM_BLOCKS x NUM_WARPS 32-lane warps per rank,
        # BUFF_SIZE of staging).  With neither, the MI355X-tuned default is
        # used: 3 slots of 512 KiB and 512 wave-channels per rank, every hop
        # of a channel on one XCD and staging kept in that XCD's L2.
        knobs = ("MINTCCL_NUM_BLOCKS", "MINTCCL_NUM_WARPS", "MINTCCL_BUFFSIZE", "MINTCCL_NSLOTS")
        reference_geometry = any(os.getenv(k) for k in knobs)
        tuned = not reference_geometry
        # tuned mode sizes slots per collective (see make_op) inside a fixed
        # budget of staging per rank
        self.auto_geometry = (tuned and buff_size_ is None and nslots is None
                              and waves_per_rank is None)
        if nslots is None:
            nslots = num_slots() if (reference_geometry or buff_size_ is not None) else TUNED_NSLOTS
        if buff_size_ is None:
            buff_size_ = buff_size() if reference_geometry else nslots * TUNED_SLOT_BUDGET
        self.buff_size, self.nslots = buff_size_, nslots
        if self.buff_size % self.nslots:
            raise ValueError("MINTCCL_BUFFSIZE must be a multiple of MINTCCL_NSLOTS")
        self.slot_bytes = self.buff_size // self.nslots
        self.protocol = protocol if protocol is not None else protocol_env()
        if placement is None:
            # the local placement deals channels to 8 XCDs: only where there are 8
            placement = placement_env() if os.getenv("MINTCCL_PLACEMENT") else (
                _lib.PLACE_LOCAL if tuned and _xcd_count(self.device) == 8 else _lib.PLACE_SPREAD)
        self.placement = placement
        if waves_per_rank is None:
            waves_per_rank = (max(1, num_blocks() * num_warps() // 2) if reference_geometry
                              else 512)
        self.waves_per_rank = waves_per_rank
        self.threads_explicit = threads_per_block is not None or bool(os.getenv("MINTCCL_THREADS"))
        self.threads_per_block = (threads_per_block if threads_per_block is not None
                                  else _env_int("MINTCCL_THREADS", 256))
        if cache_policy is None:
            cache_policy = cache_policy_env() if os.getenv("MINTCCL_CACHE") else (
                2 if self.placement == _lib.PLACE_LOCAL else 0)
        self.cache_policy = cache_policy
        if self.cache_policy == 2 and self.placement != _lib.PLACE_LOCAL:
            raise ValueError("the XCD-local cache policy needs the local placement")
        self.spin_budget = spin_budget
        self.row_fetch = row_fetch if row_fetch is not None else row_fetch_env()
        # CUs per XCD set apart for the origins of a ring broadcast / allgather:
        # an argument, MINTCCL_ORIGIN_CUS (0: none), or the tuned count
        if origin_cus is None and os.getenv("MINTCCL_ORIGIN_CUS"):
            origin_cus = _env_int("MINTCCL_ORIGIN_CUS", 0)
        self.origin_cus = origin_cus
        self._lib = _lib.lib()          # fails loudly if the extension is missing
        # slots + credit words (never more than slot_bytes / 4), zeroed: flag 0
        # and credit 0 mean "nothing yet" (2_sendrecv_indirect.py:59-60).
        if self.buff_size % 256:
            raise ValueError("staging size must be a multiple of 256 bytes")
        # (and the words thread blocks claim their seats through, behind them)
        self.rank_stride = self.buff_size + max(4096, self.slot_bytes // 4) + _lib.TICKET_BYTES
        # Whole multiples of 16 KiB between the ranks' staging: with ranks 18 or
        # 20 KiB further apart than that the 8 x 256 MiB reduce-scatter takes 10 -
        # 13 % longer (the slots of the ranks then fall differently onto the
        # channels and sets of the L2 that holds them).
        self.rank_stride = (self.rank_stride + 16383) // 16384 * 16384
        self.staging = torch.zeros(self.world_size * self.rank_stride, dtype=torch.uint8,
                                   device=self.device)
        self.status = torch.zeros(_lib.STATUS_WORDS, dtype=torch.int64, device=self.device)
        self.stats = None              # set to a zeroed int64[(hops + 1) * 8] tensor to collect wait accounting
        self.epoch = 0
        self._last_protocol = None
        # Launches that are captured into a HIP graph and replayed cannot carry
        # their epoch as an argument: with device_epoch (or MINTCCL_DEVICE_EPOCH=1)
        # it lives in device memory and every launch is preceded by a tiny
        # kernel that advances it (and clears staging when it starts over).
        if device_epoch is None:
            device_epoch = bool(os.getenv("MINTCCL_DEVICE_EPOCH", ""))
        # (two words: the epoch, and the protocol of the launch before - the
        # kernel that advances the epoch also decides, on the device, whether
        # an LL128 launch that follows a Simple one needs the slots cleared)
        self.epoch_word = (torch.zeros(2, dtype=torch.int32, device=self.device)
                           if device_epoch else None)
        self._tls = threading.local()
        self._pending: dict = {}
        self._mailbox: dict = {}
        self.last_grid = 0

    # ---- MPI-like surface -------------------------------------------------
    def Get_size(self) -> int:
        return self.world_size

    def Get_rank(self) -> int:
        r = getattr(self._tls, "rank", None)
        if r is None:
            raise RuntimeError("no current rank: use `with comm.rank(r):`")
        return r

    @contextlib.contextmanager
    def rank(self, r: int):
        if not 0 <= r < self.world_size:
            raise ValueError(f"rank {r} outside world of {self.world_size}")
        prev = getattr(self._tls, "rank", None)
        self._tls.rank = r
        try:
            yield self
        finally:
            self._tls.rank = prev

    def run(self, fn) -> None:
        """SPMD helper: ``fn(rank)`` for every rank in turn (like mpirun)."""
        for r in range(self.world_size):
            with self.rank(r):
                fn(r)

    def staging_ptr(self, r: int) -> int:
        return self.staging.data_ptr() + r * self.rank_stride

    # pointer mailbox (send_ptr / recv_ptr, common.py:22-38)
    def send_ptr(self, ptr: int, peer: int) -> None:
        self._mailbox.setdefault((self.Get_rank(), peer), []).append(ptr)

    def recv_ptr(self, peer: int) -> int:
        return self._mailbox[(peer, self.Get_rank())].pop(0)

    # ---- collective registration -------------------------------------------
    def post(self, key: str, needed: set, info) -> dict | None:
        """Record this rank's arguments; return all of them once the ranks in
        ``needed`` have posted."""
        slot = self._pending.setdefault(key, {})
        r = self.Get_rank()
        if r in slot:
            raise RuntimeError(f"rank {r} called {key} twice before the others joined")
        slot[r] = info
        if set(slot) >= needed:
            del self._pending[key]
            return slot
        return None

    # ---- launch -------------------------------------------------------------
    def make_op(self, op: int, dtype: int, count_bytes: int, inputs: dict, outputs: dict,
                ring: list[int], root: int = 0, row_stride: int = 0, route_len: int = 0,
                protocol: int | None = None, skip_origin: bool = False,
                total_bytes: int = 0) -> _lib.RingOp:
        d = _lib.RingOp()
        d.op, d.dtype, d.world = op, dtype, self.world_size
        d.protocol = self.protocol if protocol is None else protocol
        for i, r in enumerate(ring):
            d.ring[i] = r
        d.route_len, d.root = route_len, root
        for r in range(self.world_size):
            d.input[r] = inputs.get(r, NULL)
            d.output[r] = outputs.get(r, NULL)
            d.staging[r] = self.staging_ptr(r)
        d.staging_bytes = self.rank_stride
        d.count_bytes, d.row_stride, d.total_bytes = count_bytes, row_stride, total_bytes
        # credit words at a fixed place, whatever slot geometry a launch uses
        d.credit_offset = self.buff_size
        pipes = self.world_size if op in (_lib.OP_ALLGATHER, _lib.OP_REDUCESCATTER,
                                          _lib.OP_ALLREDUCE, _lib.OP_ALLTOALL) else 1
        if op == _lib.OP_ALLREDUCE:
            pipes *= 2            # a slot is shared by (pipeline, phase): two phases
        tree = op in (_lib.OP_TREE_BROADCAST, _lib.OP_TREE_REDUCE)
        if op == _lib.OP_TREE_REDUCE:
            pipes = 2             # a slot has a share per child
        hyper = op in (_lib.OP_HYPERCUBE_REDUCESCATTER, _lib.OP_HYPERCUBE_ALLGATHER)
        if hyper:
            pipes = max(1, self.world_size - 1)   # ... per stream a rank receives
        threads = self.threads_per_block
        reducing = op in (_lib.OP_REDUCE, _lib.OP_REDUCESCATTER, _lib.OP_ALLREDUCE)
        if self.auto_geometry:
            lds = (self.row_fetch == _lib.FETCH_LDS and d.protocol == _lib.PROTO_LL128
                   and reducing and threads // 64 in (4, 7))
            pairs = reducing or op in (_lib.OP_SENDRECV, _lib.OP_ALLTOALL)
            if pairs and not lds and not self.threads_explicit:
                threads = TUNED_THREADS_REDUCING
            row = count_bytes
            if op == _lib.OP_ALLREDUCE:
                row = (-(-count_bytes // self.world_size) + 15) // 16 * 16
            raw = 960 if d.protocol == _lib.PROTO_LL128 else 1024
            d.slot_bytes, d.nslots, d.waves_per_channel_group = tuned_geometry(
                op, self.world_size, route_len, threads, self.nslots, lds,
                row_blocks=max(1, -(-row // raw)), ll128=d.protocol == _lib.PROTO_LL128)
        else:
            d.slot_bytes, d.nslots = self.slot_bytes, self.nslots
            step_blocks = self.slot_bytes // 1024 // pipes
            if self.slot_bytes % 1024 or step_blocks == 0:
                raise ValueError(
                    "slot size must be a multiple of 1 KiB, at least 1 KiB per pipeline")
            # (an alltoall has twice `pipes` groups of wave-channels per rank: it
            # sends `world` rows and receives `world` rows)
            groups = 2 * pipes if op == _lib.OP_ALLTOALL else (
                1 if tree else (self.world_size if hyper else pipes))
            d.waves_per_channel_group = _largest_divisor_at_most(
                step_blocks, max(1, self.waves_per_rank // groups))
        d.threads_per_block = threads
        d.placement, d.cache_policy = self.placement, self.cache_policy
        d.row_fetch = self.row_fetch
        if self.placement == _lib.PLACE_LOCAL:
            # whole channels are dealt to the 8 XCDs; when the channel count
            # does not divide, this launch runs spread with agent-scope staging
            wpb = max(1, min(threads // 64, d.waves_per_channel_group))
            real_pipes = pipes // 2 if op == _lib.OP_ALLREDUCE else pipes
            if op == _lib.OP_ALLTOALL:
                real_pipes = self.world_size * self.world_size
            if tree:
                real_pipes = 1
            if hyper:
                real_pipes = self.world_size
            channels = real_pipes * -(-d.waves_per_channel_group // wpb)
            if channels % 8:
                d.placement = _lib.PLACE_SPREAD
                d.cache_policy = 0 if self.cache_policy == 2 else self.cache_policy
            elif self.origin_cus is not None:
                d.origin_cus = self.origin_cus
            elif op not in (_lib.OP_SENDRECV, _lib.OP_ALLTOALL) or d.protocol == _lib.PROTO_LL128:
                # (whatever the slot geometry: with the 8 slots of 512 KiB the
                # reference names an 8 x 128 MiB allgather takes 2.65 ms
                # instead of 5.07, a 64 MiB broadcast 0.18 instead of 0.32)
                npos = {_lib.OP_SENDRECV: max(route_len, 1), _lib.OP_ALLTOALL: 2}.get(
                    op, self.world_size)
                d.origin_cus = tuned_origin_cus(op, npos, channels, wpb)
        d.spin_budget = self.spin_budget
        d.status = self.status.data_ptr()
        # test hooks travel beside the descriptor (mint_ring_launch_debug)
        d.debug = None
        if skip_origin or self.stats is not None:
            d.debug = _lib.RingDebug(int(skip_origin), 0,
                                     self.stats.data_ptr() if self.stats is not None else NULL)
        return d

    def launch(self, d: _lib.RingOp) -> None:
        """Enqueue on the current stream; never synchronises."""
        # The Simple protocol writes raw payload where LL128 keeps its sector
        # tags: payload left behind by a Simple launch could pass for the tags
        # of a later LL128 launch, so the slots are cleared (a stream-ordered
        # fill) when an LL128 launch follows a Simple one on this staging.
        # With the epoch in device memory that decision is taken on the device
        # (mint_epoch_advance is told the protocol), so that a launch captured
        # into a graph takes it anew at every replay.  A launch on staging the
        # caller brought (sendrecv_buffer) is the caller's to keep to one
        # protocol or to clear.
        own_staging = d.staging[0] == self.staging_ptr(0)
        if own_staging and self.epoch_word is None:
            if d.protocol == _lib.PROTO_LL128 and self._last_protocol == _lib.PROTO_SIMPLE:
                self.staging.zero_()
                self.epoch = 0
            self._last_protocol = d.protocol
        # sector tags hold 12 bits of epoch: when the counter wraps, staging is
        # cleared (a stream-ordered fill) so that no tag of an old launch survives
        if self.epoch_word is None:
            if self.epoch >= _lib.MAX_EPOCH:
                self.staging.zero_()
                self.epoch = 0
            self.epoch += 1
            d.flag_epoch = self.epoch
        else:
            d.flag_epoch, d.epoch_ptr = 0, self.epoch_word.data_ptr()
        # (the grid of a descriptor is asked for once: a small collective is
        # host-bound, and the answer only depends on fields fixed by make_op)
        grid = getattr(d, "_grid", None)
        if grid is None:
            grid = d._grid = self._lib.mint_ring_grid_blocks(d)
        self.last_grid = grid
        with torch.cuda.device(self.device):
            stream = torch.cuda.current_stream().cuda_stream
            if self.epoch_word is not None:
                _lib.check(self._lib.mint_epoch_advance(
                    self.epoch_word.data_ptr(), self.staging.data_ptr(),
                    self.staging.numel() * self.staging.element_size(),
                    d.protocol if own_staging else -1, stream),
                    "mint_epoch_advance")
            if getattr(d, "debug", None) is not None:
                _lib.check(self._lib.mint_ring_launch_debug(d, d.debug, stream),
                           "mint_ring_launch_debug")
            else:
                _lib.check(self._lib.mint_ring_launch(d, stream), "mint_ring_launch")

    def check(self) -> None:
        """Synchronise and raise ``RingTimeout`` if a wait gave up.  Only the
        first failure is recorded; every launch queued behind it found the
        abort word set and gave up at its first wait, so the outputs of all
        launches since the last clean check are unspecified."""
        torch.cuda.synchronize(self.device)
        st = self.status.cpu().tolist()
        if st[0] != 0:
            self.status.zero_()
            who = st[1]
            # a launch that ends early can leave its seat counters behind:
            # start from cleared staging
            self.staging.zero_()
            self.epoch = 0
            if self.epoch_word is not None:
                self.epoch_word.zero_()
            if st[0] == 2:
                raise PlacementError(
                    f"a block ran on XCD {st[2]}: the local placement deals work to XCDs 0..7; "
                    "use placement spread (and cache_policy 0) on this device")
            if st[0] == 3:
                raise PlacementError(
                    "the device did not deal an eighth of the thread blocks to every XCD, so a "
                    "block of the local placement found no seat; outputs are unspecified - use "
                    "placement spread (and cache_policy 0) on this stream")
            later = (st[3] >> 32) & 0xFFFFFFFF
            raise RingTimeout(
                f"ring kernel wait ran out: pipeline {who >> 32}, position "
                f"{(who >> 16) & 0xFFFF}, wave {who & 0xFFFF}, step {st[2]}; {later} later "
                "launch(es) found the abort flag set and gave up "
                "(outputs of every launch since the last check are unspecified)")


_default_comm: VirtualComm | None = None


def get_comm() -> VirtualComm:
    """The process-wide communicator (created on first use from the env)."""
    global _default_comm
    if _default_comm is None:
        _default_comm = VirtualComm()
    return _default_comm


def set_comm(comm: VirtualComm | None) -> None:
    global _default_comm
    _default_comm = comm


def set_gpu(rank: int) -> None:
    """``common.py:10-17``: every virtual rank lives on the one visible GPU."""
    torch.set_default_device("cuda:0")


def send_ptr(ptr: int, peer: int) -> None:
    get_comm().send_ptr(ptr, peer)


def recv_ptr(peer: int) -> int:
    return get_comm().recv_ptr(peer)
