"""Pins oracle/ll128.py: closed-form maps vs independent derivations."""
import json
import os

import numpy as np
import pytest

from oracle import cref, ll128
from tests.helpers import as_bytes, uniform

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def le64(b):
    return int.from_bytes(bytes(b), "little")


def line_flags(msg, layout):
    """Flag of every line as the layout stores it (both sector tags must agree)."""
    lines = msg.reshape(-1, 128)
    if layout == ll128.LAYOUT_PAIR:
        return lines[:, 120:].copy().view("<u8").reshape(-1)
    a = lines[:, 60:64].copy().view("<u4").reshape(-1)
    b = lines[:, 124:128].copy().view("<u4").reshape(-1)
    assert (a == b).all()
    return a.astype(np.uint64)


def test_known_answer_pair_layout():
    # hand-computed from protocol.py:57-85,132-137: raw = 0..239, first line 7
    raw = np.arange(240, dtype=np.uint8)
    msg = ll128.pack(raw, 7, ll128.LAYOUT_PAIR)
    assert msg.size == 256
    assert (msg[0:120] == np.arange(0, 120)).all()
    assert le64(msg[120:128]) == 7
    assert (msg[128:240] == np.arange(128, 240)).all()
    assert (msg[240:248] == np.arange(120, 128)).all()
    assert le64(msg[248:256]) == 8


def test_known_answer_wave64_layout():
    # sector i of a block: 48 bytes of aligned vectors, 12 bytes from the tail
    # region that starts at 768, then the 32-bit tag of line i // 2
    raw = (np.arange(960) % 251).astype(np.uint8)
    msg = ll128.pack(raw, 0x1_0000_0064, ll128.LAYOUT_WAVE64)     # low 32 bits = 100
    assert msg.size == 1024
    for i in range(16):
        sec = msg[64 * i:64 * i + 64]
        assert (sec[:48] == raw[48 * i:48 * i + 48]).all()
        assert (sec[48:60] == raw[768 + 12 * i:780 + 12 * i]).all()
        assert int.from_bytes(bytes(sec[60:64]), "little") == 100 + i // 2


@pytest.mark.parametrize("seed", range(4))
def test_pair_map_equals_lane_simulation(seed):
    rng = np.random.default_rng(seed)
    raw = rng.integers(0, 256, 240, dtype=np.uint8)
    flag = int(rng.integers(1, 1 << 40)) | 1
    msg = ll128.pack(raw, flag, ll128.LAYOUT_PAIR)
    assert (msg == ll128.pair_lane_sim_pack(raw, flag)).all()
    assert (ll128.pair_lane_sim_unpack(msg) == raw).all()


@pytest.mark.parametrize("seed", range(4))
def test_wave64_map_equals_lane_simulation(seed):
    rng = np.random.default_rng(seed)
    raw = rng.integers(0, 256, 960, dtype=np.uint8)
    assert (ll128.pack(raw, 9 + seed, ll128.LAYOUT_WAVE64)
            == ll128.wave64_lane_sim_pack(raw, 9 + seed)).all()


def test_maps_are_bijections():
    for bmap, nraw in ((ll128.pair_byte_map(), 240), (ll128.wave64_byte_map(), 960)):
        data = bmap[bmap >= 0]
        assert sorted(data.tolist()) == list(range(nraw))
        assert (bmap < 0).sum() == 8 * (bmap.size // 128)      # 8 flag bytes per line


SIZES = [0, 1, 2, 15, 16, 17, 112, 119, 120, 121, 128, 239, 240, 241, 255, 256, 895, 896, 904,
         959, 960, 961, 1024, 4095, 4096, 120 * 1000, 960 * 33 + 8, (1 << 16) + 2]


@pytest.mark.parametrize("layout", [ll128.LAYOUT_PAIR, ll128.LAYOUT_WAVE64])
@pytest.mark.parametrize("n", SIZES)
def test_roundtrip_flags_size_and_c_restatement(layout, n):
    rng = np.random.default_rng(n)
    raw = rng.integers(0, 256, n, dtype=np.uint8)
    base = 1 + 7 * n
    msg = ll128.pack(raw, base, layout)
    nlines = ll128.line_count(n, layout)
    assert msg.size == nlines * 128 == ll128.packed_size(n, layout)
    if layout == ll128.LAYOUT_PAIR:
        assert nlines == -(-n // 120)
    assert (line_flags(msg, layout) == base + np.arange(nlines, dtype=np.uint64)).all()
    back, bad = ll128.unpack(msg, n, base, layout)
    assert bad == 0 and (back == raw).all()
    assert (cref.pack(raw, base, layout) == msg).all()
    back_c, bad_c = cref.unpack(msg, n, base, layout)
    assert bad_c == 0 and (back_c == raw).all()


@pytest.mark.parametrize("layout", [ll128.LAYOUT_PAIR, ll128.LAYOUT_WAVE64])
def test_wrong_flags_are_counted(layout):
    raw = np.arange(5000, dtype=np.uint8)
    msg = ll128.pack(raw, 1, layout)
    msg[3 * 128 + (120 if layout == ll128.LAYOUT_PAIR else 60)] ^= 1
    msg[0 * 128 + 127] ^= 0x80
    assert ll128.unpack(msg, raw.size, 1, layout)[1] == 2
    assert cref.unpack(msg, raw.size, 1, layout)[1] == 2
    assert ll128.unpack(msg, raw.size, 2, layout)[1] >= ll128.line_count(raw.size, layout) - 2


@pytest.mark.parametrize("layout", [ll128.LAYOUT_PAIR, ll128.LAYOUT_WAVE64])
def test_config1_roundtrip_1mib_fp16(layout):
    # benchmark configuration 1: 524,288 fp16, uniform[-1,1], seed 0; line numbers from
    # 1 (reference) and the constant "step counter 1" variant
    x = uniform(524288, -1.0, 1.0, 0)
    raw = as_bytes(x)
    for stride in (1, 0):
        msg = ll128.pack(raw, 1, layout, flag_stride=stride)
        if layout == ll128.LAYOUT_PAIR:
            assert msg.size == 8739 * 128          # 8,738 full lines + a 16-byte tail
        flags = line_flags(msg, layout)
        want = 1 + stride * np.arange(flags.size, dtype=np.uint64)
        assert (flags == want).all()
        back, bad = ll128.unpack(msg, raw.size, 1, layout, flag_stride=stride)
        assert bad == 0 and (back.view(np.uint16) == raw.view(np.uint16)).all()


def test_golden_fixture():
    """Small committed vectors written by tests/golden/make_golden.py from the
    closed forms; guards the oracle itself against accidental edits."""
    with open(os.path.join(GOLD, "ll128_vectors.json")) as f:
        gold = json.load(f)
    for case in gold["cases"]:
        raw = np.array(case["raw"], dtype=np.uint8)
        msg = ll128.pack(raw, case["flag_base"], case["layout"], case["flag_stride"])
        assert msg.tolist() == case["msg"]
        back, bad = ll128.unpack(msg, raw.size, case["flag_base"], case["layout"],
                                 case["flag_stride"])
        assert bad == 0 and back.tolist() == case["raw"]
