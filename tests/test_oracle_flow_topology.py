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


@pytest.mark.parametrize("world,nslots,steps", [
    (2, 2, 3), (3, 2, 2), (3, 3, 2), (3, 2, 4), (4, 2, 2), (4, 3, 2), (5, 2, 1), (5, 3, 2)])
def test_temporal_allgather_hands_its_credit_words_over_safely(world, nslots, steps):
    """One agent per position; the rank it serves changes from phase to phase
    and with it who posts a rank's credit word."""
    r = flowmodel.explore_temporal(world, nslots, steps)
    assert r.overwritten == 0 and r.wrong == 0 and r.deadlocks == 0 and r.finals == 1


def test_checker_catches_a_credit_word_posted_without_the_hand_over():
    # an agent that posts a rank's word before the agent that served the rank
    # in the phase before is through releases slots that are still full
    for world, nslots, steps in ((3, 2, 2), (3, 2, 3), (4, 2, 1)):
        r = flowmodel.explore_temporal(world, nslots, steps, handover=False)
        assert r.overwritten > 0


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


def test_topo_json_round_trip_in_the_reference_format(tmp_path):
    """``topo.json`` as the reference writes it (``topology.py:128-150``): a
    dict keyed by the source rank - a string once it has been through JSON -
    of ``[dst, GB/s]`` pairs.  What ``save_topology`` writes is that, and
    ``get_topology`` reads it back unchanged."""
    import json
    rng = random.Random(7)
    topo = random_topology(6, rng, p=0.7)
    topo = {s: sorted(links, key=lambda e: (-e[1], e[0])) for s, links in topo.items()}
    path = tmp_path / "topo.json"
    topology.save_topology(topo, str(path))
    doc = json.load(open(path))
    assert sorted(doc) == [str(s) for s in range(6)]
    for s, links in doc.items():
        assert all(isinstance(d, int) and isinstance(bw, float) for d, bw in links)
        assert [bw for _, bw in links] == sorted((bw for _, bw in links), reverse=True)
    assert topology.get_topology(str(path)) == topo
    assert topology.find_ring(topology.get_topology(str(path))) == topology.find_ring(topo)


def test_topo_json_written_the_reference_way_is_read(tmp_path):
    # the reference sorts every list with sorted(items, reverse=True): by
    # destination id, descending (topology.py:148), and dumps int keys
    import json
    raw = {0: [(1, 48.2), (2, 23.9), (3, 24.1)], 1: [(0, 48.2), (2, 24.0), (3, 47.9)],
           2: [(0, 23.9), (1, 24.0), (3, 48.0)], 3: [(0, 24.1), (1, 47.9), (2, 48.0)]}
    as_reference = {src: sorted(items, reverse=True) for src, items in raw.items()}
    path = tmp_path / "topo.json"
    json.dump(as_reference, open(path, "w"))
    topo = topology.get_topology(str(path))
    assert set(topo) == {0, 1, 2, 3}
    assert topo[0] == [(1, 48.2), (3, 24.1), (2, 23.9)]        # widest first
    # the ring through the three wide links and one narrow one: 0-1-3-2-0 (bottleneck 23.9)
    # against 0-1-2-3-0 (24.0) and 0-2-1-3-0 (23.9): the best bottleneck is 24.0
    ring = topology.find_ring(topo)
    assert otopo.ring_bandwidth(topo, ring) == otopo.best_ring_bandwidth(topo) == 24.0
    assert topology.find_route(0, 2, topo) == [0, 2]                   # a direct link wins
    missing = {s: [(d, bw) for d, bw in links if {s, d} != {0, 2}] for s, links in topo.items()}
    assert topology.find_route(0, 2, missing) == [0, 1, 3, 2]          # widest: min(48.2, 47.9, 48.0)


def test_get_topology_without_a_file_is_uniform(tmp_path):
    topo = topology.get_topology(str(tmp_path / "absent.json"), world_size=4)
    assert topo == topology.uniform_topology(4)
