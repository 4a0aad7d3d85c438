"""Pins oracle/ring.py: the element addition and the ring fold order."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import cref, ll128, ring
from tests.helpers import random_bits, special_values_f16

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def exact_then_round_once_f16(a_bits, b_bits):
    """binary64 holds the sum of two binary16 values exactly; one rounding."""
    a = a_bits.view(np.float16).astype(np.float64)
    b = b_bits.view(np.float16).astype(np.float64)
    with np.errstate(all="ignore"):
        return (a + b).astype(np.float16).view(np.uint16)


def exact_then_round_once_bf16(a_bits, b_bits):
    a = (a_bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    b = (b_bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    with np.errstate(all="ignore"):
        s = a + b                      # exact unless exponents are > 52 apart,
    # in which case the smaller operand is below half an ulp of bf16 anyway
    # round binary64 -> bf16 (8 significant bits, emin -126) to nearest even
    # with frexp / rint, then read the bits off the (exactly representable) value
    with np.errstate(all="ignore"):
        m, e = np.frexp(s)                                   # s = m * 2**e, 0.5 <= |m| < 1
        e = np.maximum(e, -125)                              # subnormal quantum 2**-133
        q = np.ldexp(np.rint(np.ldexp(s, 8 - e)), e - 8)     # rint: ties to even
        q32 = q.astype(np.float32)                           # exact, or overflow to inf
    out = (q32.view(np.uint32) >> 16).astype(np.uint16)
    big = np.abs(q) >= 2.0 ** 128
    out[big] = np.where(q[big] > 0, 0x7F80, 0xFF80).astype(np.uint16)
    out[np.isnan(s)] = 0x7FC0
    return out


def test_add_f16_is_one_correct_rounding():
    a, b = random_bits(400000, 16, 1), random_bits(400000, 16, 2)
    got = ring.add_rn(a, b, "f16").view(np.uint16)
    want = exact_then_round_once_f16(a, b)
    assert ring.same_values(got, want, "f16")


def test_add_bf16_is_one_correct_rounding():
    a, b = random_bits(400000, 16, 3), random_bits(400000, 16, 4)
    got = ring.add_rn(a, b, "bf16").view(np.uint16)
    want = exact_then_round_once_bf16(a, b)
    assert ring.same_values(got, want, "bf16")


@pytest.mark.parametrize("dt", ["f16", "bf16"])
def test_add_matches_integer_softfloat(dt):
    a, b = random_bits(1 << 20, 16, 5), random_bits(1 << 20, 16, 6)
    assert ring.same_values(ring.add_rn(a, b, dt), cref.add(a, b, dt), dt)
    sp = special_values_f16()
    aa, bb = np.meshgrid(sp, sp)
    aa, bb = aa.reshape(-1).copy(), bb.reshape(-1).copy()
    assert ring.same_values(ring.add_rn(aa, bb, dt), cref.add(aa, bb, dt), dt)


def test_add_f16_exhaustive_near_subnormals():
    # every pair of the 2048 smallest magnitudes of both signs: subnormal
    # results, cancellation to +0, -0 + -0 = -0
    mags = np.arange(0, 1100, dtype=np.uint16)
    vals = np.concatenate([mags, mags | 0x8000])
    aa, bb = np.meshgrid(vals, vals)
    aa, bb = aa.reshape(-1).copy(), bb.reshape(-1).copy()
    got = ring.add_rn(aa, bb, "f16").view(np.uint16)
    assert (got == cref.add(aa, bb, "f16").view(np.uint16)).all()
    assert (got == exact_then_round_once_f16(aa, bb)).all()


@pytest.mark.parametrize("dt,tdt", [("f16", torch.float16), ("bf16", torch.bfloat16),
                                    ("f32", torch.float32)])
def test_add_matches_torch_cpu(dt, tdt):
    bits = 32 if dt == "f32" else 16
    a, b = random_bits(200000, bits, 7), random_bits(200000, bits, 8)
    iv = torch.int32 if bits == 32 else torch.int16
    ta = torch.from_numpy(a.view(np.int32 if bits == 32 else np.int16)).view(tdt)
    tb = torch.from_numpy(b.view(np.int32 if bits == 32 else np.int16)).view(tdt)
    want = (ta + tb).view(iv).numpy()
    assert ring.same_values(ring.add_rn(a, b, dt), want, dt)


def test_hand_computed_fold_order():
    # 2048 has ulp 2 in binary16: 2048 + 1 -> 2048 (tie to even), so the
    # position of the large value in the fold is visible in the result
    f = lambda *v: [np.array([x], dtype=np.float16).view(np.uint8) for x in v]
    rows = f(2048.0, 1.0, 1.0)
    as_f = lambda raw: float(raw.view(np.float16)[0])
    assert as_f(ring.fold(rows, [0, 1, 2], "f16")) == 2048.0   # (2048+1)+1
    assert as_f(ring.fold(rows, [1, 2, 0], "f16")) == 2050.0   # (1+1)+2048


def test_hand_computed_fold_order_exact_values():
    f = lambda *v: [np.array([x], dtype=np.float16).view(np.uint8) for x in v]
    as_f = lambda raw: float(raw.view(np.float16)[0])
    rows = f(2048.0, 1.0, 1.0)
    # acc = 1; 2048 + 1 = 2049 -> 2048; 1 + 2048 = 2049 -> 2048
    assert as_f(ring.fold(rows, [2, 0, 1], "f16")) == 2048.0


def test_reduce_order_follows_ring_from_root():
    with open(os.path.join(GOLD, "fold_vectors.json")) as f:
        gold = json.load(f)
    # element 0 by hand: root 0 -> ((2048+1)+1)+0.5 = 2048; root 1 -> ((1+1)+0.5)+2048 = 2050
    by_root = {c["root"]: c for c in gold["cases"]}
    assert np.array(by_root[0]["result_f16_bits"], dtype=np.uint16).view(np.float16)[0] == 2048.0
    assert np.array(by_root[1]["result_f16_bits"], dtype=np.uint16).view(np.float16)[0] == 2050.0
    for c in gold["cases"]:
        xs = [np.array(r, dtype=np.uint16).view(np.uint8) for r in c["rows_f16_bits"]]
        out = ring.reduce(xs, c["root"], "f16")
        assert out[c["root"]].view(np.uint16).tolist() == c["result_f16_bits"]
        for r in range(4):
            if r != c["root"]:
                assert (out[r] == xs[r]).all()       # non-roots keep their data


def test_hand_computed_tree_order():
    """Binary tree over the node order: (own + first subtree) + second subtree."""
    f = lambda *v: [np.array([x], dtype=np.float16).view(np.uint8) for x in v]
    as_f = lambda raw: float(raw.view(np.float16)[0])
    # three nodes: (2048 + 1) + 1 = 2048 where (1 + 1) + 2048 would give 2050
    assert as_f(ring.tree_fold(f(2048.0, 1.0, 1.0), [0, 1, 2], "f16")) == 2048.0
    # first child before second: (2048 + 1) -> 2048, + 1.5 -> 2050;
    # the other way round (2048 + 1.5) -> 2050, + 1 = 2051 -> 2052
    assert as_f(ring.tree_fold(f(2048.0, 1.0, 1.5), [0, 1, 2], "f16")) == 2050.0
    assert as_f(ring.tree_fold(f(2048.0, 1.5, 1.0), [0, 1, 2], "f16")) == 2052.0
    # five nodes: node 1 has children 3 and 4.  Tree: (2048 + ((1 + 1) + 0)) + 0 = 2050;
    # the ring order ((((2048 + 1) + 0) + 1) + 0) loses both ones: 2048
    rows = f(2048.0, 1.0, 0.0, 1.0, 0.0)
    assert as_f(ring.tree_fold(rows, [0, 1, 2, 3, 4], "f16")) == 2050.0
    assert as_f(ring.fold(rows, [0, 1, 2, 3, 4], "f16")) == 2048.0
    # the node order is the ring turned to the root
    assert ring.tree_nodes([0, 2, 1, 3, 4, 0], 1) == [1, 3, 4, 0, 2]
    xs = [rows[i] for i in (3, 0, 4, 1, 2)]        # rank r holds the value of node [1,3,4,0,2].index(r)
    out = ring.tree_reduce(xs, 1, "f16", [0, 2, 1, 3, 4, 0])
    assert as_f(out[1]) == 2050.0
    assert all((out[r] == xs[r]).all() for r in (0, 2, 3, 4))


@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
def test_tree_reduce_properties(dt):
    bits = 32 if dt == "f32" else 16
    # two ranks: one commutative addition, the same as the ring's
    a, b = random_bits(4000, bits, 31), random_bits(4000, bits, 32)
    x = [a.view(np.uint8), b.view(np.uint8)]
    assert ring.same_values(ring.tree_reduce(x, 1, dt)[1], ring.reduce(x, 1, dt)[1], dt)
    # small integers add exactly in any order: the tree and the ring agree with the plain sum
    rng = np.random.default_rng(5)
    vals = [rng.integers(-8, 9, 1000).astype(np.float32) for _ in range(7)]
    if dt == "f32":
        raw = [v.view(np.uint8) for v in vals]
    elif dt == "f16":
        raw = [v.astype(np.float16).view(np.uint8) for v in vals]
    else:
        raw = [(v.view(np.uint32) >> 16).astype(np.uint16).view(np.uint8) for v in vals]
    for root in (0, 3, 6):
        t = ring.tree_reduce(raw, root, dt)[root]
        assert ring.same_values(t, ring.reduce(raw, root, dt)[root], dt)
        assert np.array_equal(ring.to_float64(t, dt), np.sum(vals, axis=0, dtype=np.float64))


def test_hand_computed_hypercube_order():
    """Recursive halving: corner i adds the partner across the highest bit
    first.  f16 near 2048 has a spacing of 2 and ties go to the even
    significand: 2048 + 1 -> 2048, 2048 + 1.5 -> 2050, 2050 + 1 -> 2052,
    2052 + 3 -> 2056."""
    as_f = lambda raw, r, n: float(raw.view(np.float16).reshape(n, -1)[r, 0])

    def buffers(n, row, values):
        """Rank r's (n, 1) buffer: ``values[r]`` in row ``row``, zero elsewhere."""
        out = []
        for r in range(n):
            b = np.zeros((n, 1), dtype=np.float16)
            b[row, 0] = values[r]
            out.append(b.view(np.uint8).reshape(-1))
        return out

    # four corners, row 0: (x0 + x2) + (x1 + x3) = (2048 + 1.5) + (1 + 0) = 2050 + 1 -> 2052;
    # the ring ((2048 + 1) + 1.5) + 0, the binary tree (2048 + (1 + 0)) + 1.5 and halving
    # from the lowest bit (2048 + 1) + (1.5 + 0) all give 2050
    xs = buffers(4, 0, [2048.0, 1.0, 1.5, 0.0])
    assert as_f(ring.hypercube_reducescatter(xs, "f16")[0], 0, 4) == 2052.0
    assert as_f(ring.reducescatter(xs, "f16")[0], 0, 4) == 2050.0
    assert float(ring.tree_fold([x[:2] for x in xs], [0, 1, 2, 3], "f16").view(np.float16)[0]) == 2050.0
    # row 3: (x3 + x1) + (x2 + x0) = (2048 + 1.5) + (0 + 1) -> 2052
    xs = buffers(4, 3, [1.0, 1.5, 0.0, 2048.0])
    assert as_f(ring.hypercube_reducescatter(xs, "f16")[3], 3, 4) == 2052.0
    # eight corners, row 0: ((x0 + x4) + (x2 + x6)) + ((x1 + x5) + (x3 + x7))
    # = ((2048 + 1.5) + (1 + 0)) + ((1 + 1) + (1 + 0)) = (2050 + 1 -> 2052) + 3 -> 2056;
    # the ring loses the ones: 2048 +1 +1 +1 -> 2048, + 1.5 -> 2050, + 1 -> 2052
    xs = buffers(8, 0, [2048.0, 1.0, 1.0, 1.0, 1.5, 1.0, 0.0, 0.0])
    assert as_f(ring.hypercube_reducescatter(xs, "f16")[0], 0, 8) == 2056.0
    assert as_f(ring.reducescatter(xs, "f16")[0], 0, 8) == 2052.0
    # row 5 = 0b101: ((x5 + x1) + (x7 + x3)) + ((x4 + x0) + (x6 + x2)), the same values
    # moved to the corners that play these parts
    vals = [0.0] * 8
    for part, v in zip((5, 1, 7, 3, 4, 0, 6, 2), (2048.0, 1.5, 1.0, 0.0, 1.0, 1.0, 1.0, 0.0)):
        vals[part] = v
    assert as_f(ring.hypercube_reducescatter(buffers(8, 5, vals), "f16")[5], 5, 8) == 2056.0
    # corners follow the ring: with ring 0 2 1 3 corner 1 is rank 2, so rank 2's row is
    # (x[rank 2] + x[rank 3]) + (x[rank 0] + x[rank 1])  (corners 1, 3, 0, 2)
    xs = buffers(4, 2, [1.0, 0.0, 2048.0, 1.5])
    out = ring.hypercube_reducescatter(xs, "f16", [0, 2, 1, 3, 0])
    assert as_f(out[2], 2, 4) == 2052.0
    # only row r of rank r changes
    assert all((out[r] == xs[r]).all() for r in (0, 1, 3))
    # the operator's own account of the order (nested pairs of corner numbers)
    from mintccl_amd import hypercube
    assert hypercube.order(4, 0) == ((0, 2), (1, 3))
    assert hypercube.order(8, 0) == (((0, 4), (2, 6)), ((1, 5), (3, 7)))
    assert hypercube.order(8, 5) == (((5, 1), (7, 3)), ((4, 0), (6, 2)))


@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
def test_hypercube_properties(dt):
    bits = 32 if dt == "f32" else 16
    # two ranks: one commutative addition, the same as the ring's
    x = [random_bits(2 * 3000, bits, 41 + r).view(np.uint8) for r in range(2)]
    for mine, ringed in zip(ring.hypercube_reducescatter(x, dt), ring.reducescatter(x, dt)):
        assert ring.same_values(mine, ringed, dt)
    # small integers add exactly in any order
    rng = np.random.default_rng(6)
    for n in (4, 8):
        vals = [rng.integers(-8, 9, (n, 500)).astype(np.float32) for _ in range(n)]
        if dt == "f32":
            raw = [v.view(np.uint8).reshape(-1) for v in vals]
        elif dt == "f16":
            raw = [v.astype(np.float16).view(np.uint8).reshape(-1) for v in vals]
        else:
            raw = [(v.view(np.uint32) >> 16).astype(np.uint16).view(np.uint8).reshape(-1) for v in vals]
        for perm in (None, [3, 1, 0, 2] + list(range(4, n)) + [3]):
            mine = ring.hypercube_reducescatter(raw, dt, perm)
            ringed = ring.reducescatter(raw, dt, perm)
            for r in range(n):
                assert ring.same_values(mine[r], ringed[r], dt)
                got = ring.to_float64(mine[r], dt).reshape(n, -1)[r]
                assert np.array_equal(got, np.sum([v[r] for v in vals], axis=0, dtype=np.float64))
    with pytest.raises(ValueError):
        ring.hypercube_reducescatter([x[0]] * 3, dt)


def test_hypercube_allgather_is_allgather():
    rng = np.random.default_rng(7)
    for n in (1, 2, 4, 8):
        xs = [rng.integers(0, 256, n * 96, dtype=np.uint8) for _ in range(n)]
        for perm in (None, list(reversed(range(n))) + [n - 1]):
            mine = ring.hypercube_allgather(xs, perm)
            for a, b in zip(mine, ring.allgather(xs)):
                assert np.array_equal(a, b)
    with pytest.raises(ValueError):
        ring.hypercube_allgather([xs[0]] * 6)


def test_fold_order_with_a_permuted_ring():
    ring_ = [0, 2, 1, 3, 0]
    assert ring.fold_order(ring_, 1) == [1, 3, 0, 2]
    assert ring.fold_order(ring_, 0) == [0, 2, 1, 3]
    assert ring.fold_order(ring.identity_ring(8), 5) == [5, 6, 7, 0, 1, 2, 3, 4]


def test_two_ranks_is_one_commutative_add():
    a, b = random_bits(5000, 16, 11), random_bits(5000, 16, 12)
    x = [a.view(np.uint8), b.view(np.uint8)]
    r0 = ring.reduce(x, 0, "f16")[0]
    r1 = ring.reduce(x, 1, "f16")[1]
    assert ring.same_values(r0, r1, "f16")
    assert ring.same_values(r0, ring.add_rn(a, b, "f16"), "f16")


@pytest.mark.parametrize("dt", ring.DTYPES)
def test_fold_stays_within_half_ulp_steps_of_exact_sum(dt):
    n_ranks, n = 8, 4096
    g = torch.Generator().manual_seed(1)
    xs = [torch.randn(n, generator=g).to({"f16": torch.float16, "bf16": torch.bfloat16,
                                          "f32": torch.float32}[dt]) for _ in range(n_ranks)]
    raw = [x.view(torch.uint8).numpy() for x in xs]
    got = ring.to_float64(ring.reduce(raw, 0, dt)[0], dt)
    exact = sum(ring.to_float64(r, dt) for r in raw)
    eps = {"f16": 2.0 ** -11, "bf16": 2.0 ** -8, "f32": 2.0 ** -24}[dt]
    bound = (n_ranks - 1) * eps * sum(np.abs(ring.to_float64(r, dt)) for r in raw)
    assert (np.abs(got - exact) <= bound + 1e-30).all()


@pytest.mark.parametrize("dt", ring.DTYPES)
@pytest.mark.parametrize("world", [2, 3, 8])
def test_wire_walk_equals_closed_form(dt, world):
    item = ring.ITEMSIZE[dt]
    n = 1237
    rng = np.random.default_rng(world)
    tdt = {"f16": np.float16, "bf16": None, "f32": np.float32}[dt]

    def rand(count):
        v = rng.standard_normal(count).astype(np.float32)
        if dt == "bf16":
            return (v.view(np.uint32) >> 16).astype(np.uint16).view(np.uint8)
        return v.astype(tdt).view(np.uint8)

    xs = [rand(n) for _ in range(world)]
    for layout in (ll128.LAYOUT_PAIR, ll128.LAYOUT_WAVE64):
        assert all((a == b).all() for a, b in zip(ring.reduce(xs, 1, dt),
                                                  ring.reduce_wire(xs, 1, dt, layout=layout)))
    rows = [rand(world * n) for _ in range(world)]
    assert all((a == b).all() for a, b in zip(ring.reducescatter(rows, dt),
                                              ring.reducescatter_wire(rows, dt)))
    assert all((a == b).all() for a, b in zip(ring.broadcast(xs, world - 1),
                                              ring.broadcast_wire(xs, world - 1)))
    assert n * item == xs[0].size


def test_copy_collectives_are_identities():
    world, n = 4, 100
    rng = np.random.default_rng(0)
    rows = [rng.integers(0, 256, world * n, dtype=np.uint8) for _ in range(world)]
    out = ring.allgather(rows)
    for r in range(world):
        for c in range(world):
            assert (out[r].reshape(world, n)[c] == rows[c].reshape(world, n)[c]).all()
    out = ring.sendrecv(rows, 2, 0)
    assert (out[0] == rows[2]).all() and (out[1] == rows[1]).all()
    rs = ring.reducescatter([r.view(np.uint8) for r in rows], "f16")
    for r in range(world):
        for c in range(world):
            if r != c:      # only row r of rank r changes
                assert (rs[r].reshape(world, n)[c] == rows[r].reshape(world, n)[c]).all()


def test_allreduce_chunks_and_order():
    # 4 ranks, 20 f16 values: rows of 16 bytes (8 values): chunks [0:8], [8:16], [16:20], []
    assert ring.allreduce_row_bytes(40, 4) == 16
    rows = [[2048.0, 1.0, 2048.0, 1.0], [1.0, 1.0, 1.0, 1.0], [1.0, 2048.0, 1.0, 2048.0],
            [1.0, 1.0, 1.0, 1.0]]
    xs = []
    for r in range(4):
        v = np.ones(20, dtype=np.float16)
        v[0:8] = rows[r][0]; v[8:16] = rows[r][1]; v[16:20] = rows[r][2]
        xs.append(v.view(np.uint8))
    out = ring.allreduce(xs, "f16")
    got = out[0].view(np.float16)
    assert got[0] == 2048.0 and got[8] == 2048.0 and got[16] == 2052.0   # same hand values as reducescatter
    assert all((o == out[0]).all() for o in out)
    # against reducescatter + allgather of the padded buffer
    world, n = 3, 1000
    rng = np.random.default_rng(0)
    xs = [rng.standard_normal(n).astype(np.float16).view(np.uint8) for _ in range(world)]
    row = ring.allreduce_row_bytes(2 * n, world)
    padded = [np.concatenate([x, np.zeros(world * row - x.size, np.uint8)]) for x in xs]
    want = ring.allgather(ring.reducescatter(padded, "f16"))[0][:2 * n]
    assert all((o == want).all() for o in ring.allreduce(xs, "f16"))


@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("world,n", [(8, 1000), (3, 481), (4, 7), (2, 960)])
def test_torch_cpu_walk_equals_the_numpy_walk(dt, world, n):
    """The PyTorch-CPU walk that bench.py times as the CPU baseline gives the
    bits of the numpy restatement (which the tests above pin), through the
    wire format, for a permuted ring as well."""
    import torch
    from oracle import torch_ring
    g = torch.Generator().manual_seed(world * 1000 + n)
    bufs = [torch.randn(world, n, generator=g).to(torch_ring.TORCH_DT[dt]) for _ in range(world)]
    raw = [b.view(torch.uint8).numpy().reshape(-1) for b in bufs]
    rings = [None, list(reversed(range(world))) + [world - 1]]
    for rg in rings:
        got = torch_ring.reducescatter_wire(bufs, dt, ring=rg, flag_base=(1 << 32) - 5)
        want = ring.reducescatter_wire(raw, dt, ring=rg, flag_base=(1 << 32) - 5)
        assert ring.reducescatter(raw, dt, ring=rg)[0].tobytes() == want[0].tobytes()
        for r in range(world):
            assert np.array_equal(got[r].view(torch.uint8).numpy().reshape(-1), want[r]), r


def test_alltoall_is_the_transpose_of_rows():
    # hand-written: 3 ranks, rows of two bytes; rank s row d = (10 s + d) twice
    xs = [np.array([[10 * s + d] * 2 for d in range(3)], dtype=np.uint8).reshape(-1) for s in range(3)]
    out = ring.alltoall(xs)
    assert out[0].tolist() == [0, 0, 10, 10, 20, 20]
    assert out[1].tolist() == [1, 1, 11, 11, 21, 21]
    assert out[2].tolist() == [2, 2, 12, 12, 22, 22]
    rng = np.random.default_rng(3)
    xs = [rng.integers(0, 256, 5 * 37, dtype=np.uint8) for _ in range(5)]
    twice = ring.alltoall(ring.alltoall(xs))
    assert all(np.array_equal(a, b) for a, b in zip(twice, xs))          # an involution
    assert sum(int(x.sum()) for x in xs) == sum(int(x.sum()) for x in ring.alltoall(xs))
