"""Element arithmetic and ring-collective results on the CPU.  Test
infrastructure, never shipped.

Arithmetic.  The reference reduces with PTX ``add.f16x2`` on packed halves
(``primitive.py:232-247``): IEEE-754 binary16 addition, round to nearest even,
subnormals kept, no saturation.  ``add_rn`` restates that for f16 and extends
it, one rounding per addition, to bf16 and f32.

* f16: ``numpy.float16`` addition (computed in binary32, rounded once more to
  binary16; the second rounding is innocuous because 24 >= 2*11 + 2).
* bf16: operands widened to binary32, one binary32 addition, then round to
  nearest even on the bit pattern; a NaN result is the canonical 0x7FC0.
  (24 >= 2*8 + 2, same argument.)
* f32: ``numpy.float32`` addition.

Pinning of ``add_rn``: ``tests/test_oracle_ring`` checks it against an exact
binary64 sum rounded once (f16, bf16), against the integer-only soft-float
adder in ``ll128_ref.c`` on random and special bit patterns, and against
torch-CPU addition.  NaN payloads are not part of the contract: two results
are equal if both are NaN (``same_values``).

Collectives.  ``ring`` is the rank sequence ``[r0, ..., r_{N-1}, r0]`` the
reference's ``find_ring`` returns (``topology.py:56-93``); data moves
``ring[i] -> ring[i+1]`` because every rank hands its staging pointer to the
previous rank and writes into the next one's (``5_reduce.py:114-115``,
``7_reducescatter.py:95-96``).

* ``reduce``: the root sends its own values unreduced, every other rank adds
  its own values to what arrives and forwards, the root stores what comes
  back (``5_reduce.py:70-89``; ``comp_ll128`` computes ``own + received``,
  ``protocol.py:150-155``).  So with the ring rotated to start at the root,
  ``acc = x[root]; acc = rn(x[r_k] + acc)`` for k = 1..N-1.
* ``reducescatter``: chunk ``c`` of the ``(N, n)`` buffer is reduced the same
  way with rank ``c`` as root and lands in row ``c`` of rank ``c``
  (``7_reducescatter.py:23-34,54-73``).
* ``allgather``: row ``c`` of every rank becomes rank ``c``'s row ``c``
  (``6_allgather.py:56-74``).  ``broadcast`` / ``sendrecv``: destination bytes
  become source bytes (``4_broadcast.py:61-72``, ``2_sendrecv_indirect.py:80-90``).

Pinning of the fold order: N = 2 is a single commutative addition; the
2048 + 1 + 1 family distinguishes this order from reverse and tree orders;
the result stays within (N-1) half-ulp steps of the exact sum.  The reference
pins its own results only by run-time equality with NCCL, which cannot run
here, and note that NCCL's ring order differs from this one - the order
restated is what the cited kernel lines compute.
"""
from __future__ import annotations

import numpy as np

from . import ll128

DTYPES = ("f16", "bf16", "f32")
ITEMSIZE = {"f16": 2, "bf16": 2, "f32": 4}


def _bytes(a) -> np.ndarray:
    return np.ascontiguousarray(a).view(np.uint8).reshape(-1)


def add_rn(a, b, dtype: str) -> np.ndarray:
    """Elementwise ``rn(a + b)`` on raw bytes; returns raw bytes (uint8)."""
    a, b = _bytes(a), _bytes(b)
    if a.size != b.size or a.size % ITEMSIZE[dtype]:
        raise ValueError("operand sizes do not match the dtype")
    with np.errstate(all="ignore"):
        if dtype == "f16":
            return _bytes(a.view(np.float16) + b.view(np.float16))
        if dtype == "f32":
            return _bytes(a.view(np.float32) + b.view(np.float32))
        if dtype == "bf16":
            fa = (a.view(np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)
            fb = (b.view(np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)
            s = (fa + fb).astype(np.float32)
            bits = s.view(np.uint32)
            lsb = (bits >> np.uint32(16)) & np.uint32(1)
            rounded = ((bits + np.uint32(0x7FFF) + lsb) >> np.uint32(16)).astype(np.uint16)
            rounded[np.isnan(s)] = np.uint16(0x7FC0)
            return _bytes(rounded)
    raise ValueError(f"unknown dtype {dtype}")


def to_float64(raw, dtype: str) -> np.ndarray:
    raw = _bytes(raw)
    if dtype == "f16":
        return raw.view(np.float16).astype(np.float64)
    if dtype == "f32":
        return raw.view(np.float32).astype(np.float64)
    if dtype == "bf16":
        return (raw.view(np.uint16).astype(np.uint32) << np.uint32(16)).view(
            np.float32).astype(np.float64)
    raise ValueError(dtype)


def same_values(a, b, dtype: str) -> bool:
    """Bit equality, except that any NaN equals any NaN."""
    a, b = _bytes(a), _bytes(b)
    if a.size != b.size:
        return False
    w = {2: np.uint16, 4: np.uint32}[ITEMSIZE[dtype]]
    ne = a.view(w) != b.view(w)
    if not ne.any():
        return True
    fa, fb = to_float64(a, dtype), to_float64(b, dtype)
    return bool(np.all(~ne | (np.isnan(fa) & np.isnan(fb))))


def identity_ring(world: int) -> list[int]:
    return list(range(world)) + [0]


def fold_order(ring: list[int], root: int) -> list[int]:
    """Ranks in the order their values enter the accumulator."""
    cyc = ring[:-1]
    i = cyc.index(root)
    return cyc[i:] + cyc[:i]


def fold(rows: list, order: list[int], dtype: str) -> np.ndarray:
    acc = _bytes(rows[order[0]]).copy()
    for r in order[1:]:
        acc = add_rn(rows[r], acc, dtype)      # own + received
    return acc


def reduce(xs: list, root: int, dtype: str, ring: list[int] | None = None) -> list:
    """xs[r] = rank r's buffer (bytes).  Returns the buffers after the call."""
    ring = ring or identity_ring(len(xs))
    out = [_bytes(x).copy() for x in xs]
    out[root] = fold(xs, fold_order(ring, root), dtype)
    return out


def reducescatter(xs: list, dtype: str, ring: list[int] | None = None) -> list:
    """xs[r] = rank r's (N, n) buffer as bytes (row-major)."""
    n_ranks = len(xs)
    ring = ring or identity_ring(n_ranks)
    rows = [_bytes(x).reshape(n_ranks, -1) for x in xs]
    out = [r.copy() for r in rows]
    for c in range(n_ranks):
        out[c][c] = fold([rows[r][c] for r in range(n_ranks)], fold_order(ring, c), dtype)
    return [o.reshape(-1) for o in out]


def allgather(xs: list) -> list:
    n_ranks = len(xs)
    rows = [_bytes(x).reshape(n_ranks, -1) for x in xs]
    out = [r.copy() for r in rows]
    for r in range(n_ranks):
        for c in range(n_ranks):
            out[r][c] = rows[c][c]
    return [o.reshape(-1) for o in out]


def allreduce_row_bytes(nbytes: int, world: int) -> int:
    """Bytes of one chunk: the buffer is cut into ``world`` rows of whole
    16-byte vectors; the last rows may be short or empty."""
    return (-(-nbytes // world) + 15) // 16 * 16


def allreduce(xs: list, dtype: str, ring: list[int] | None = None) -> list:
    """Chunk c is folded in ring order starting from rank c's own value
    (the reduce-scatter order) and every rank ends up with every folded chunk.
    The reference only plans this collective (``README.md:23``); the order is
    the one its reduce-scatter uses."""
    n_ranks = len(xs)
    ring = ring or identity_ring(n_ranks)
    raw = [_bytes(x) for x in xs]
    total = raw[0].size
    row = allreduce_row_bytes(total, n_ranks)
    out = np.empty(total, dtype=np.uint8)
    for c in range(n_ranks):
        lo, hi = min(c * row, total), min((c + 1) * row, total)
        if hi > lo:
            out[lo:hi] = fold([r[lo:hi] for r in raw], fold_order(ring, c), dtype)
    return [out.copy() for _ in xs]


def alltoall(xs: list) -> list:
    """xs[s] = rank s's ``(N, n)`` buffer (bytes).  Returns every rank's output:
    row s of rank d is row d of rank s (MPI_Alltoall; the reference plans it
    as ``9_alltoall.py``, ``README.md:24,50``, and holds no code for it).
    Pinned by definition: a transpose of whole rows, bit-exact copies; applied
    twice it gives the input back."""
    n_ranks = len(xs)
    rows = [_bytes(x).reshape(n_ranks, -1) for x in xs]
    return [np.concatenate([rows[s][d] for s in range(n_ranks)]) for d in range(n_ranks)]


def broadcast(xs: list, root: int) -> list:
    return [_bytes(xs[root]).copy() for _ in xs]


def tree_nodes(ring: list[int], root: int) -> list[int]:
    """Ranks in node order of the binary tree laid over the ring turned to the
    root: node h has parent (h - 1) // 2 and children 2h + 1, 2h + 2."""
    return fold_order(ring, root)


def tree_fold(rows: list, nodes: list[int], dtype: str, h: int = 0) -> np.ndarray:
    """What node h passes to its parent: (own + first subtree) + second
    subtree, one rounding per addition."""
    acc = _bytes(rows[nodes[h]]).copy()
    for c in (2 * h + 1, 2 * h + 2):
        if c < len(nodes):
            acc = add_rn(acc, tree_fold(rows, nodes, dtype, c), dtype)
    return acc


def tree_reduce(xs: list, root: int, dtype: str, ring: list[int] | None = None) -> list:
    """Reduce up a binary tree ("Tree / Binary Tree" is an open item of the
    reference's roadmap, ``README.md:52-55``; the reference holds no code for
    it, so the order of the additions is this build's definition - parity with
    the reference is unpinned by construction).  The building blocks are the
    reference's: ``comp_ll128`` (``protocol.py:142-156``) adds own + received
    with one rounding.  Pinned: against hand-computed values that tell this
    order from the ring's and from (first + second) + own; equal to
    ``reduce`` for N = 2; within (N - 1) half-ulp steps of the exact sum."""
    ring = ring or identity_ring(len(xs))
    out = [_bytes(x).copy() for x in xs]
    out[root] = tree_fold(xs, tree_nodes(ring, root), dtype)
    return out


def hypercube_nodes(ring: list[int]) -> list[int]:
    """Ranks in corner order of the hypercube laid over the ring: corner i is
    the i-th rank of the ring."""
    return list(ring[:-1])


def hypercube_reducescatter(xs: list, dtype: str, ring: list[int] | None = None) -> list:
    """Reduce-scatter by recursive halving ("Hypercube" is an open item of the
    reference's roadmap, ``README.md:52-55``; the reference holds no code for
    it, so the order of the additions is this build's definition - parity with
    the reference is unpinned by construction).  xs[r] = rank r's (N, n) buffer
    as bytes, N = 2^d.  Played as the exchanges themselves: every corner starts
    with its own values of all N rows; in exchange k = 0 .. d-1 corner i and
    corner i ^ D, D = N >> (k + 1), split the rows both still hold - a row of
    corner c stays with the one of the two whose bit D equals c's - and the
    keeper's partial sum becomes keeper's + partner's, one rounding
    (``comp_ll128``, ``protocol.py:142-156``).  After d exchanges corner i holds
    row i of its rank.  Buffers as ``reducescatter``: only row r of rank r
    changes.  Pinned: against hand-computed values that tell this order from
    the ring's and from the binary tree's; equal to ``reducescatter`` for
    N = 2; within (N - 1) half-ulp steps of the exact sum."""
    n_ranks = len(xs)
    if n_ranks < 1 or n_ranks & (n_ranks - 1):
        raise ValueError("a hypercube has 2^d corners")
    ring = ring or identity_ring(n_ranks)
    corners = hypercube_nodes(ring)
    rows = [_bytes(x).reshape(n_ranks, -1) for x in xs]
    # held[i][c]: corner i's partial sum of the row that belongs to corner c
    held = [{c: rows[corners[i]][corners[c]].copy() for c in range(n_ranks)}
            for i in range(n_ranks)]
    span = n_ranks >> 1
    while span:
        after = []
        for i in range(n_ranks):
            partner = i ^ span
            after.append({c: add_rn(held[i][c], held[partner][c], dtype)
                          for c in held[i] if (c & span) == (i & span)})
        held, span = after, span >> 1
    out = [r.copy() for r in rows]
    for i in range(n_ranks):
        assert list(held[i]) == [i]
        out[corners[i]][corners[i]] = held[i][i]
    return [o.reshape(-1) for o in out]


def hypercube_allgather(xs: list, ring: list[int] | None = None) -> list:
    """Allgather by recursive doubling: the exchanges of
    ``hypercube_reducescatter`` backwards, every corner handing its partner all
    rows it holds.  Bytes only move, so the result is ``allgather``'s; played
    out to check that the exchanges reach every corner."""
    n_ranks = len(xs)
    if n_ranks < 1 or n_ranks & (n_ranks - 1):
        raise ValueError("a hypercube has 2^d corners")
    corners = hypercube_nodes(ring or identity_ring(n_ranks))
    rows = [_bytes(x).reshape(n_ranks, -1) for x in xs]
    held = [{i: rows[corners[i]][corners[i]]} for i in range(n_ranks)]
    span = 1
    while span < n_ranks:
        held = [{**held[i], **held[i ^ span]} for i in range(n_ranks)]
        span <<= 1
    out = [r.copy() for r in rows]
    for i in range(n_ranks):
        for c, row in held[i].items():
            out[corners[i]][corners[c]] = row
    return [o.reshape(-1) for o in out]


def sendrecv(xs: list, src: int, dst: int) -> list:
    out = [_bytes(x).copy() for x in xs]
    out[dst] = _bytes(xs[src]).copy()
    return out


# --------------------------------------------------------------------------
# The same collectives pushed through the wire format, hop by hop.  This is
# what the device does and what the CPU baseline times: every hop packs the
# outgoing lines with their flags, the receiver checks the flags, unpacks and
# (for reductions) adds its own values.
# --------------------------------------------------------------------------
def _hop(payload: np.ndarray, flag_base: int, layout: int) -> np.ndarray:
    msg = ll128.pack(payload, flag_base, layout)
    raw, bad = ll128.unpack(msg, payload.size, flag_base, layout)
    if bad:
        raise AssertionError(f"{bad} lines arrived with a wrong flag")
    return raw


def reduce_wire(xs: list, root: int, dtype: str, ring: list[int] | None = None,
                layout: int = ll128.LAYOUT_WAVE64, flag_base: int = 1) -> list:
    ring = ring or identity_ring(len(xs))
    order = fold_order(ring, root)
    out = [_bytes(x).copy() for x in xs]
    acc = _bytes(xs[order[0]]).copy()
    for r in order[1:]:
        acc = add_rn(xs[r], _hop(acc, flag_base, layout), dtype)
    out[root] = _hop(acc, flag_base, layout)
    return out


def reducescatter_wire(xs: list, dtype: str, ring: list[int] | None = None,
                       layout: int = ll128.LAYOUT_WAVE64, flag_base: int = 1) -> list:
    n_ranks = len(xs)
    ring = ring or identity_ring(n_ranks)
    rows = [_bytes(x).reshape(n_ranks, -1) for x in xs]
    out = [r.copy() for r in rows]
    for c in range(n_ranks):
        order = fold_order(ring, c)
        acc = rows[order[0]][c].copy()
        for r in order[1:]:
            acc = add_rn(rows[r][c], _hop(acc, flag_base, layout), dtype)
        out[c][c] = _hop(acc, flag_base, layout)
    return [o.reshape(-1) for o in out]


def broadcast_wire(xs: list, root: int, ring: list[int] | None = None,
                   layout: int = ll128.LAYOUT_WAVE64, flag_base: int = 1) -> list:
    ring = ring or identity_ring(len(xs))
    order = fold_order(ring, root)
    out = [_bytes(x).copy() for x in xs]
    cur = _bytes(xs[root]).copy()
    for r in order[1:]:
        cur = _hop(cur, flag_base, layout)
        out[r] = cur.copy()
    return out
