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

``LAYOUT_WAVE64`` - the format the HIP kernels use for staging.  On MI355X a
128-byte store does not become visible as a whole (64-byte sectors do), so the
8 flag bytes of a line are spent as one 32-bit tag per 64-byte sector::

    line = [0,60) payload | [60,64) tag | [64,124) payload | [124,128) tag

where tag = low 32 bits of the line's flag, little endian.  One 64-lane
wavefront moves a *block* of 8 lines (16 sectors) with one 16-byte access per
lane: 960 raw bytes <-> 1024 message bytes.  Lane ``l`` with ``l % 4 != 3``
carries the aligned raw vector number ``l - l // 4`` (0..47); the flag lane of
sector ``i`` (``l = 4 i + 3``) carries raw bytes ``[768 + 12 i, 780 + 12 i)``
and the tag.  So, inside block ``b`` (first line number ``f = base + 8 b``)::

    msg[64 i      : 64 i + 48] = raw[48 i : 48 i + 48]
    msg[64 i + 48 : 64 i + 60] = raw[768 + 12 i : 780 + 12 i]
    msg[64 i + 60 : 64 i + 64] = LE32(f + i // 2)          i = 0..15

A buffer whose size is not a multiple of the unit is zero padded: the pair
layout packs ``ceil(n / 120)`` lines, the wave64 layout ``ceil(n / 960)``
whole blocks.  (The reference drops the tail, ``2_sendrecv_indirect.py:65,74``;
the intent - deliver every byte - is what is restated.)

Pinning.  The closed-form maps below are checked in ``tests/test_oracle_ll128``
against (i) per-lane simulations written independently from the register
moves in the cited lines, (ii) the hand-computed known answer for raw = 0..239,
f = 7, (iii) the integer-only C restatement ``ll128_ref.c``, and (iv) the
invariants ``unpack(pack(x)) == x``, flags where the layout puts them in every
line, packed size.  The reference holds no golden vectors for this path.
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
SECTOR_BYTES = 64                  # what becomes visible as a whole on MI355X
BLOCK_SECTORS = 16
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
    """message byte -> raw byte, or -(1 + line) for a byte of that line's tag."""
    m = np.empty(BLOCK_MSG, dtype=np.int64)
    for i in range(BLOCK_SECTORS):
        m[64 * i:64 * i + 48] = np.arange(48 * i, 48 * i + 48)
        m[64 * i + 48:64 * i + 60] = np.arange(768 + 12 * i, 780 + 12 * i)
        m[64 * i + 60:64 * i + 64] = -(1 + i // 2)
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


def _put_flags(lines: np.ndarray, flags: np.ndarray, layout: int) -> None:
    if layout == LAYOUT_PAIR:
        lines[:, 120:128] = flags.astype("<u8").view(np.uint8).reshape(-1, 8)
    else:
        tag = (flags & np.uint64(0xFFFFFFFF)).astype("<u4").view(np.uint8).reshape(-1, 4)
        lines[:, 60:64] = tag
        lines[:, 124:128] = tag


def _count_bad_flags(lines: np.ndarray, flags: np.ndarray, layout: int) -> int:
    if layout == LAYOUT_PAIR:
        got = lines[:, 120:128].copy().view("<u8").reshape(-1)
        return int(np.count_nonzero(got != flags))
    want = (flags & np.uint64(0xFFFFFFFF)).astype(np.uint32)
    a = lines[:, 60:64].copy().view("<u4").reshape(-1)
    b = lines[:, 124:128].copy().view("<u4").reshape(-1)
    return int(np.count_nonzero((a != want) | (b != want)))


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
    _put_flags(lines, flags, layout)
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
    bad = _count_bad_flags(lines[:nlines], _flags(nlines, flag_base, flag_stride), layout)
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
    lanes load the aligned 16-byte vector ``lane - lane // 4``; the flag lane
    of sector ``i`` loads 16 bytes starting 4 bytes before its 12 and shifts."""
    msg = np.zeros(1024, dtype=np.uint8)
    for lane in range(64):
        i, q = divmod(lane, 4)
        if q != 3:
            vec = lane - i
            msg[lane * 16:lane * 16 + 16] = raw960[vec * 16:vec * 16 + 16]
        else:
            start = 768 + 12 * i - 4
            loaded = raw960[start:start + 16]
            msg[lane * 16:lane * 16 + 12] = loaded[4:16]
            tag = (first_flag + (i // 2) * flag_stride) & 0xFFFFFFFF
            msg[lane * 16 + 12:lane * 16 + 16] = np.frombuffer(
                int(tag).to_bytes(4, "little"), dtype=np.uint8)
    return msg
