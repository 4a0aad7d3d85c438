"""Brute-force ring / route search.  Test infrastructure, never shipped.

Restates the *intent* of ``topology.py:23-93``: ``find_ring`` returns a
Hamiltonian cycle through node 0 whose smallest edge bandwidth is as large as
possible; ``find_route`` returns a widest simple path (a direct link wins).
Both enumerate everything, so they are only for small graphs.

Pinning: by definition (exhaustive maximum).  Which of several equally good
cycles the reference returns depends on its heap order (``topology.py:69-91``);
that tie-break is *parity unpinned* - it cannot be imported here - and does
not arise for the uniform virtual-rank graph, where reading the heap priority
(longer path first, then smaller node id, strict ``>`` at ``:79``) gives the
identity ring ``[0, 1, ..., N-1, 0]``.
"""
from __future__ import annotations

import itertools


def _bw(topo, u, v):
    for d, bw in topo[u]:
        if d == v:
            return bw
    return None


def best_ring_bandwidth(topo) -> float:
    n = len(topo)
    best = 0.0
    for perm in itertools.permutations(range(1, n)):
        cyc = (0,) + perm + (0,)
        widths = [_bw(topo, a, b) for a, b in zip(cyc, cyc[1:])]
        if None not in widths:
            best = max(best, min(widths))
    return best


def ring_bandwidth(topo, ring) -> float:
    widths = [_bw(topo, a, b) for a, b in zip(ring, ring[1:])]
    return 0.0 if None in widths else min(widths)


def best_route_bandwidth(topo, src, dst) -> float:
    best = 0.0
    nodes = [x for x in topo if x not in (src, dst)]
    for k in range(len(nodes) + 1):
        for mid in itertools.permutations(nodes, k):
            path = (src,) + mid + (dst,)
            widths = [_bw(topo, a, b) for a, b in zip(path, path[1:])]
            if None not in widths:
                best = max(best, min(widths))
    return best
