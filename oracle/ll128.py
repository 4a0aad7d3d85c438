"""LL128 line codec on the CPU (numpy).  Test infrastructure, never shipped.

A *line* is 128 message bytes: 120 payload bytes followed by an 8-byte
little-endian flag (reference ``protocol.py:42-48``: ``BYTES_LL128_MSG`` = 128,
``BYTES_LL128_RAW`` = 120).  Two layouts are restated here.

``LAYOUT_PAIR`` - the reference's wire format.  An 8-lane workgroup moves a
pair of lines per step (``ITERS_PER_SEND`` = 2): 240 raw bytes <-> 256 message
bytes.  From ``load_ll128`` (``protocol.py:57-85``) and ``send_ll128``
(``protocol.py:132-137``), with ``f`` the 1-based number of the first line::

    msg[  0:112] = raw[  0:112]      lanes 0-6, registers (v0, v1)
    msg[112:120] = raw[112:120]      lane 7, v0
    msg[120:128] = LE64(f)           lane 7, v1
    msg[128:240] = raw[128:240]      lanes 0-6, (v2, v3)
    msg[240:248] = raw[120:128]      lane 7, v2 (upper half of its one load)
    msg[248:256] = LE64(f + 1)       lane 7, v3

``save_ll128`` (``protocol.py:87-100``) is the inverse.  Line numbers start at
1 and are unique over a transfer (``2_sendrecv_indirect.py:61,93``).

``LAYOUT_WAVE64`` - the format the HIP kernels use for staging.  One 64-lane
wavefront moves a *block* of 8 lines with one 16-byte access per lane:
960 raw bytes <-> 1024 message bytes.  Lane ``l`` with ``l % 8 != 7`` carries
the aligned raw vector number ``l - l // 8`` (0..55); the flag lane of line
``j`` (``l = 8 j + 7``) carries raw bytes ``[896 + 8 j, 904 + 8 j)`` and the
flag.  So, inside block ``b`` (first line number ``f = base + 8 b``)::

    msg[128 j      : 128 j + 112] = raw[112 j : 112 j + 112]
    msg[128 j + 112: 128 j + 120] = raw[896 + 8 j : 904 + 8 j]
    msg[128 j + 120: 128 j + 128] = LE64(f + j)            j = 0..7

A buffer whose size is not a multiple of the unit is zero padded: the pair
layout packs ``ceil(n / 120)`` lines, the wave64 layout ``ceil(n / 960)``
whole blocks.  (The reference drops the tail, ``2_sendrecv_indirect.py:65,74``;
the intent - deliver every byte - is what is restated.)

Pinning.  The closed-form maps below are checked in ``tests/test_oracle_ll128``
against (i) per-lane simulations written independently from the register
moves in the cited lines, (ii) the hand-computed known answer for raw = 0..239,
f = 7, (iii) the integer-only C restatement ``ll128_ref.c``, and (iv) the
invariants ``unpack(pack(x)) == x``, flags at bytes 120..127 of every line,
packed size.  The reference holds no golden vectors for this path.
"""
from __future__ import annotations

import numpy as np

LINE_BYTES = 128          # protocol.py:47  BYTES_LL128_MSG
LINE_PAYLOAD = 120        # protocol.py:48  BYTES_LL128_RAW
FLAG_BYTES = 8            # protocol.py:43  PAYLOAD_FLAG_THREAD
LANE_BYTES = 16           # protocol.py:42  PAYLOAD_WORK_THREAD
LANES_PER_LINE = 8        # protocol.py:44  WORKGROUP_SIZE

PAIR_RAW = 2 * LINE_PAYLOAD        # 240
PAIR_MSG = 2 * LINE_BYTES          # 256
BLOCK_LINES = 8                    # lines per 64-lane access
BLOCK_RAW = BLOCK_LINES * LINE_PAYLOAD   # 960
BLOCK_MSG = BLOCK_LINES * LINE_BYTES     # 1024

LAYOUT_PAIR = 0
LAYOUT_WAVE64 = 1


# --------------------------------------------------------------------------
# closed-form byte maps: message byte -> raw byte (>= 0) or -(1 + line) = flag
# --------------------------------------------------------------------------
def pair_byte_map() -> np.ndarray:
    m = np.empty(PAIR_MSG, dtype=np.int64)
    m[0:120] = np.arange(0, 120)
    m[120:128] = -1
    m[128:240] = np.arange(128, 240)
    m[240:248] = np.arange(120, 128)
    m[248:256] = -2
    return m


def wave64_byte_map() -> np.ndarray:
    m = np.empty(BLOCK_MSG, dtype=np.int64)
    for j in range(BLOCK_LINES):
        m[128 * j:128 * j + 112] = np.arange(112 * j, 112 * j + 112)
        m[128 * j + 112:128 * j + 120] = np.arange(896 + 8 * j, 904 + 8 * j)
        m[128 * j + 120:128 * j + 128] = -(1 + j)
    return m


def _unit(layout: int):
    if layout == LAYOUT_PAIR:
        return PAIR_RAW, PAIR_MSG, 2, pair_byte_map()
    if layout == LAYOUT_WAVE64:
        return BLOCK_RAW, BLOCK_MSG, BLOCK_LINES, wave64_byte_map()
    raise ValueError(f"unknown LL128 layout {layout}")


def line_count(nbytes: int, layout: int) -> int:
    """Number of lines a packed buffer of ``nbytes`` raw bytes holds."""
    if layout == LAYOUT_PAIR:
        return -(-nbytes // LINE_PAYLOAD)
    if layout == LAYOUT_WAVE64:
        return -(-nbytes // BLOCK_RAW) * BLOCK_LINES
    raise ValueError(f"unknown LL128 layout {layout}")


def packed_size(nbytes: int, layout: int) -> int:
    return line_count(nbytes, layout) * LINE_BYTES


def _flags(nlines: int, flag_base: int, flag_stride: int) -> np.ndarray:
    return (np.uint64(flag_base)
            + np.arange(nlines, dtype=np.uint64) * np.uint64(flag_stride))


def pack(raw, flag_base: int = 1, layout: int = LAYOUT_PAIR,
         flag_stride: int = 1) -> np.ndarray:
    """raw bytes -> LL128 message bytes.

    Line ``L`` (0-based) carries flag ``flag_base + L * flag_stride``:
    ``flag_stride`` = 1, ``flag_base`` = 1 gives the reference's line numbers
    (``2_sendrecv_indirect.py:61``); ``flag_stride`` = 0 stamps every line with
    the same step counter.
    """
    raw = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
    n = raw.size
    uraw, umsg, ulines, bmap = _unit(layout)
    nlines = line_count(n, layout)
    nunits = -(-nlines // ulines)
    padded = np.zeros(nunits * uraw, dtype=np.uint8)
    padded[:n] = raw
    units = padded.reshape(nunits, uraw)
    msg = np.zeros((nunits, umsg), dtype=np.uint8)
    data = bmap >= 0
    msg[:, data] = units[:, bmap[data]]
    flags = np.zeros(nunits * ulines, dtype=np.uint64)
    flags[:nlines] = _flags(nlines, flag_base, flag_stride)
    lines = msg.reshape(nunits * ulines, LINE_BYTES)
    lines[:, LINE_PAYLOAD:] = flags.astype("<u8").view(np.uint8).reshape(-1, 8)
    return lines[:nlines].reshape(-1).copy()


def unpack(msg, nbytes: int, flag_base: int = 1, layout: int = LAYOUT_PAIR,
           flag_stride: int = 1):
    """LL128 message bytes -> (raw bytes[nbytes], number of lines whose flag
    differs from the expected one)."""
    msg = np.ascontiguousarray(msg).view(np.uint8).reshape(-1)
    uraw, umsg, ulines, bmap = _unit(layout)
    nlines = line_count(nbytes, layout)
    if msg.size < nlines * LINE_BYTES:
        raise ValueError("message buffer too small")
    nunits = -(-nlines // ulines)
    full = np.zeros(nunits * umsg, dtype=np.uint8)
    full[:nlines * LINE_BYTES] = msg[:nlines * LINE_BYTES]
    lines = full.reshape(nunits * ulines, LINE_BYTES)
    got = lines[:nlines, LINE_PAYLOAD:].copy().view("<u8").reshape(-1)
    bad = int(np.count_nonzero(got != _flags(nlines, flag_base, flag_stride)))
    units = full.reshape(nunits, umsg)
    raw = np.zeros((nunits, uraw), dtype=np.uint8)
    data = bmap >= 0
    raw[:, bmap[data]] = units[:, data]
    return raw.reshape(-1)[:nbytes].copy(), bad


# --------------------------------------------------------------------------
# per-lane simulations (independent derivations used only to pin the maps)
# --------------------------------------------------------------------------
def _u64(b: np.ndarray) -> int:
    return int.from_bytes(bytes(b), "little")


def _b64(v: int) -> np.ndarray:
    return np.frombuffer(int(v).to_bytes(8, "little"), dtype=np.uint8)


def pair_lane_sim_pack(raw240: np.ndarray, flag: int) -> np.ndarray:
    """One pair step, lane by lane: ``load_ll128`` then ``send_ll128``
    (``protocol.py:57-85,132-137``)."""
    raw = np.zeros(256, dtype=np.uint8)          # lane 7's load reads [112,128)
    raw[:240] = raw240
    msg = np.zeros(256, dtype=np.uint8)
    for lane in range(8):
        v0 = _u64(raw[lane * 16:lane * 16 + 8])
        v1 = _u64(raw[lane * 16 + 8:lane * 16 + 16])
        if lane != 7:
            v2 = _u64(raw[128 + lane * 16:128 + lane * 16 + 8])
            v3 = _u64(raw[128 + lane * 16 + 8:128 + lane * 16 + 16])
        else:
            v2, v1, v3 = v1, flag, flag + 1
        msg[lane * 16:lane * 16 + 8] = _b64(v0)
        msg[lane * 16 + 8:lane * 16 + 16] = _b64(v1)
        msg[128 + lane * 16:128 + lane * 16 + 8] = _b64(v2)
        msg[128 + lane * 16 + 8:128 + lane * 16 + 16] = _b64(v3)
    return msg


def pair_lane_sim_unpack(msg256: np.ndarray) -> np.ndarray:
    """One pair step, lane by lane: the loads of ``recv_ll128`` then
    ``save_ll128`` (``protocol.py:102-130,87-100``)."""
    raw = np.zeros(240, dtype=np.uint8)
    for lane in range(8):
        v0 = msg256[lane * 16:lane * 16 + 8]
        v1 = msg256[lane * 16 + 8:lane * 16 + 16]
        v2 = msg256[128 + lane * 16:128 + lane * 16 + 8]
        v3 = msg256[128 + lane * 16 + 8:128 + lane * 16 + 16]
        if lane != 7:
            raw[lane * 16:lane * 16 + 8] = v0
            raw[lane * 16 + 8:lane * 16 + 16] = v1
            raw[128 + lane * 16:128 + lane * 16 + 8] = v2
            raw[128 + lane * 16 + 8:128 + lane * 16 + 16] = v3
        else:
            raw[112:120] = v0
            raw[120:128] = v2
    return raw


def wave64_lane_sim_pack(raw960: np.ndarray, first_flag: int,
                         flag_stride: int = 1) -> np.ndarray:
    """One block, lane by lane, the way a 64-lane wavefront does it: data
    lanes load the aligned 16-byte vector ``lane - lane // 8``; the flag lane
    of line ``j`` loads vector ``56 + j // 2`` and keeps its half ``j % 2``."""
    msg = np.zeros(1024, dtype=np.uint8)
    for lane in range(64):
        j, k = divmod(lane, 8)
        if k != 7:
            vec = lane - j
            msg[lane * 16:lane * 16 + 16] = raw960[vec * 16:vec * 16 + 16]
        else:
            vec = 56 + j // 2
            half = raw960[vec * 16 + 8 * (j % 2):vec * 16 + 8 * (j % 2) + 8]
            msg[lane * 16:lane * 16 + 8] = half
            msg[lane * 16 + 8:lane * 16 + 16] = _b64(first_flag + j * flag_stride)
    return msg
