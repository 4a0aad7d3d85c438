"""Flow-control model checker and ring / route search."""
import itertools
import random

import pytest

from oracle import flowmodel, topology as otopo
from mintccl_amd import topology


@pytest.mark.parametrize("hops,nslots,steps,lines", [
    (1, 1, 4, 2), (1, 2, 5, 2), (2, 1, 4, 2), (2, 2, 5, 2), (2, 3, 5, 2), (3, 2, 4, 2),
    (3, 3, 5, 1), (3, 1, 3, 3)])
def test_credit_protocol_is_safe_and_live(hops, nslots, steps, lines):
    r = flowmodel.explore(hops, nslots, steps, lines)
    assert r.overwritten == 0 and r.wrong == 0 and r.deadlocks == 0 and r.finals >= 1


def test_checker_catches_early_credit():
    # the reference posts its credit at the start of every round
    # (3_sendrecv_buffer.py:49-52): a fast sender then overwrites lines that
    # have not been taken, or the receiver waits for a flag that is gone
    r = flowmodel.explore(2, 2, 5, 2, post_early=True)
    assert r.overwritten > 0 and r.deadlocks > 0


def test_checker_reports_a_lost_line_as_a_deadlock():
    r = flowmodel.explore(2, 2, 4, 2, drop=(0, 1, 1))
    assert r.deadlocks > 0 and r.finals == 0


def random_topology(n, rng, p=0.8):
    topo = {i: [] for i in range(n)}
    for a, b in itertools.combinations(range(n), 2):
        if rng.random() < p:
            bw = float(rng.choice([5, 10, 25, 50]))
            topo[a].append((b, bw))
            topo[b].append((a, bw))
    return {k: sorted(v, key=lambda e: (-e[1], e[0])) for k, v in topo.items()}


@pytest.mark.parametrize("seed", range(12))
def test_find_ring_maximises_the_bottleneck(seed):
    rng = random.Random(seed)
    n = rng.choice([3, 4, 5, 6])
    topo = random_topology(n, rng)
    ring = topology.find_ring(topo)
    best = otopo.best_ring_bandwidth(topo)
    if best == 0.0:
        assert ring == []
    else:
        assert ring[0] == ring[-1] == 0 and sorted(ring[:-1]) == list(range(n))
        assert otopo.ring_bandwidth(topo, ring) == best


@pytest.mark.parametrize("n", [1, 2, 3, 4, 8])
def test_uniform_topology_gives_the_identity_ring(n):
    assert topology.find_ring(topology.uniform_topology(n)) == list(range(n)) + [0]


@pytest.mark.parametrize("seed", range(12))
def test_find_route_is_widest(seed):
    rng = random.Random(100 + seed)
    n = rng.choice([3, 4, 5, 6])
    topo = random_topology(n, rng, p=0.6)
    src, dst = rng.sample(range(n), 2)
    route = topology.find_route(src, dst, topo)
    best = otopo.best_route_bandwidth(topo, src, dst)
    if best == 0.0:
        assert route == []
        return
    assert route[0] == src and route[-1] == dst and len(set(route)) == len(route)
    direct = otopo._bw(topo, src, dst)
    if direct is not None:
        assert route == [src, dst]          # a direct link wins (topology.py:30)
    else:
        assert otopo.ring_bandwidth(topo, route) == best
    short = topology.find_route(src, dst, topo, shortest=True)
    assert short[0] == src and short[-1] == dst and len(short) <= len(route)


def test_find_plan():
    assert topology.find_plan([0, 2, 1, 3, 0], 1) == (2, 3)
    assert topology.find_plan([0, 1, 0], 0) == (1, 1)
