"""Ring and route search (host only).

Mirrors ``topology.py:18-93`` of the reference: the same type aliases and the
same two entry points, built to their stated intent - ``find_ring`` returns a
Hamiltonian cycle through node 0 that maximises the bottleneck bandwidth,
``find_route`` the widest path (direct link first, or the shortest path on
request).  The virtual ranks of one GPU form a uniform complete graph, for
which the ring is ``[0, 1, ..., N-1, 0]``.  The bandwidth probe of
``topology.py:96-150`` needs several GPUs and is not part of this build;
``get_topology`` returns the uniform graph or loads a ``topo.json`` of the
reference's format ``{src: [[dst, GB/s], ...]}``.
"""
from __future__ import annotations

import heapq
import json
import os

Topology = dict[int, list[tuple[int, float]]]   # src -> [(dst, bandwidth)], widest first
Route = list[int]
Plan = tuple[int, int]                           # prev, next


def uniform_topology(world_size: int, bandwidth: float = 1.0) -> Topology:
    return {s: [(d, bandwidth) for d in range(world_size) if d != s]
            for s in range(world_size)}


def get_topology(topo: str = "topo.json", world_size: int | None = None) -> Topology:
    if os.path.exists(topo):
        with open(topo) as f:
            raw = json.load(f)
        return {int(s): sorted(((int(d), float(bw)) for d, bw in items),
                               key=lambda e: (-e[1], e[0]))
                for s, items in raw.items()}
    if world_size is None:
        from .common import get_comm
        world_size = get_comm().world_size
    return uniform_topology(world_size)


def find_route(src: int, dst: int, topo: Topology | None = None,
               shortest: bool = False) -> Route:
    """Widest path src -> dst (``topology.py:23-53``); a direct link wins;
    ``shortest=True`` minimises hops, widest among equals.  ``[]`` if none."""
    if topo is None:
        topo = get_topology()
    if src == dst:
        return [src]
    if any(v == dst for v, _ in topo[src]):
        return [src, dst]
    # best-first on (hops, -width) or (-width, hops)
    best: dict[int, tuple] = {}
    heap = [((0, -float("inf")) if shortest else (-float("inf"), 0), src, [src])]
    while heap:
        key, u, path = heapq.heappop(heap)
        if u == dst:
            return path
        if u in best and best[u] <= key:
            continue
        best[u] = key
        width = -key[1] if shortest else -key[0]
        for v, bw in topo[u]:
            if v in path:
                continue
            w = min(width, bw)
            k = (len(path), -w) if shortest else (-w, len(path))
            heapq.heappush(heap, (k, v, path + [v]))
    return []


def find_ring(topo: Topology | None = None) -> Route:
    """Hamiltonian cycle through node 0 with the largest bottleneck bandwidth
    (``topology.py:56-93``); node 0 appears first and last; ``[]`` if none.
    Among equally good cycles the lexicographically smallest is returned,
    which for a uniform graph is the identity ring."""
    if topo is None:
        topo = get_topology()
    n = len(topo)
    if n == 1:
        return [0, 0]
    nbr = {u: sorted(topo[u]) for u in topo}
    best_cycle: Route = []
    best_bw = 0.0

    def extend(path: list[int], width: float) -> None:
        nonlocal best_cycle, best_bw
        u = path[-1]
        if len(path) == n:
            for v, bw in nbr[u]:
                if v == path[0] and min(width, bw) > best_bw:
                    best_bw, best_cycle = min(width, bw), path + [path[0]]
            return
        for v, bw in nbr[u]:
            if v in path or min(width, bw) <= best_bw:
                continue
            extend(path + [v], min(width, bw))

    extend([0], float("inf"))
    return best_cycle


def find_plan(ring: Route, rank: int) -> Plan:
    """(prev, next) of ``rank`` on the ring (the indexing every reference host
    function repeats, e.g. ``7_reducescatter.py:91-96``)."""
    n = len(ring) - 1
    pos = ring.index(rank)
    return ring[(pos - 1) % n], ring[(pos + 1) % n]
