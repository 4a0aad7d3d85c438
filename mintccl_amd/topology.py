"""Ring and route search (host only).

Mirrors ``topology.py:18-93`` of the reference: the same type aliases and the
same two entry points, built to their stated intent - ``find_ring`` returns a
Hamiltonian cycle through node 0 that maximises the bottleneck bandwidth,
``find_route`` the widest path (direct link first, or the shortest path on
request).  The virtual ranks of one GPU form a uniform complete graph, for
which the ring is ``[0, 1, ..., N-1, 0]``.

``get_topology`` loads a ``topo.json`` of the reference's format
(``topology.py:128-150``: ``{"src": [[dst, GB/s], ...], ...}``, keys turned
into strings by ``json.dump``), or returns the uniform graph; ``save_topology``
writes that format; ``probe_topology`` is the reference's measurement pass
(``get_p2p_speed`` for every pair, ``topology.py:96-126,135-148``) run between
the buffers of virtual ranks, where a "link" is a copy inside one GPU's HBM
(the peer-to-peer copies between GPUs that the reference times need more than
one GPU).
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


def save_topology(topo: Topology, path: str = "topo.json") -> None:
    """Write ``topo`` the way the reference persists it (``topology.py:148-149``):
    one entry per source, its links as ``[dst, bandwidth]`` pairs, widest
    first (the reference's own ``sorted(items, reverse=True)`` orders by
    destination id; the stated intent - "sorted", widest first - is what is
    written, and readers accept any order)."""
    doc = {str(src): [[int(d), float(bw)] for d, bw in sorted(links, key=lambda e: (-e[1], e[0]))]
           for src, links in sorted(topo.items())}
    with open(path, "w") as f:
        json.dump(doc, f)


def get_p2p_speed(src: int, dst: int, size: int = 33554432, comm=None) -> float:
    """GB/s of a ``size``-byte copy from virtual rank ``src`` to virtual rank
    ``dst`` (``topology.py:96-126``; there a ``cudaMemcpyPeerAsync`` between two
    GPUs, here the library's own copy kernel between two buffers of one GPU),
    timed with events on the current stream."""
    import torch

    from . import primitive
    from .common import get_comm
    comm = comm if comm is not None else get_comm()
    a = torch.empty(size, dtype=torch.uint8, device=comm.device)
    b = torch.empty(size, dtype=torch.uint8, device=comm.device)
    primitive.copy128(a, b)                                  # first touch
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    primitive.copy128(a, b)
    stop.record()
    torch.cuda.synchronize(comm.device)
    return size / (start.elapsed_time(stop) / 1e3) / 1e9


def probe_topology(world_size: int | None = None, path: str | None = None, comm=None) -> Topology:
    """Measure every pair once, both directions get the same figure
    (``topology.py:135-148``), and persist the result if ``path`` is given."""
    from .common import get_comm
    comm = comm if comm is not None else get_comm()
    world_size = world_size if world_size is not None else comm.world_size
    topo: Topology = {s: [] for s in range(world_size)}
    for s in range(world_size):
        for d in range(s + 1, world_size):
            bw = get_p2p_speed(s, d, comm=comm)
            topo[s].append((d, bw))
            topo[d].append((s, bw))
    topo = {s: sorted(links, key=lambda e: (-e[1], e[0])) for s, links in topo.items()}
    if path is not None:
        save_topology(topo, path)
    return topo


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
