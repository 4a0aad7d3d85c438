"""GPU parity, through the C ABI: copy, LL128 codec, element sum vs the oracle."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import ll128, ring
from tests.helpers import as_bytes, random_bits, special_values_f16, uniform

pytestmark = pytest.mark.gpu

SIZES = [0, 1, 15, 16, 17, 119, 120, 121, 240, 241, 959, 960, 961, 4096, 65536 + 2,
         960 * 1000 + 8, (1 << 20) + 7]


def dev_bytes(a: np.ndarray, dev) -> torch.Tensor:
    return torch.from_numpy(a.copy()).to(dev)


def test_device_is_mi355x_shaped(lib):
    cu, xcd, wave = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    assert lib.mint_device_info(cu, xcd, wave) == 0
    # 8 XCDs, and the probe found every aligned group of 8 blocks on 8 different ones
    assert wave.value == 64 and cu.value > 0 and xcd.value == 8


def test_blocks_are_dealt_round_robin_over_xcds(lib, dev):
    """What the local placement relies on: consecutive blocks go to consecutive
    XCDs, so every aligned group of 8 covers all 8 - from whichever XCD block
    0 lands on, which changes with the hardware queue behind the stream."""
    from mintccl_amd import primitive
    cu, xcd, wave = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    lib.mint_device_info(cu, xcd, wave)
    n = xcd.value

    def check():
        m = primitive.xcd_map(64, dev).cpu().tolist()
        assert m == [(m[0] + i) % n for i in range(64)]
        return m[0]

    starts = {check()}
    other = torch.cuda.Stream(device=dev)
    with torch.cuda.stream(other):
        src = torch.zeros(1 << 20, dtype=torch.uint8, device=dev)
        primitive.copy128(src, torch.empty_like(src), blocks=3, threads=256)
        starts.add(check())
    other.synchronize()
    starts.add(check())          # the default stream may have moved to another queue
    assert starts <= set(range(n))


@pytest.mark.parametrize("n", [0, 1, 16, 1000, (1 << 20) + 5, (64 << 20) + 16])
def test_copy_simple(dev, n):
    from mintccl_amd import primitive
    g = torch.Generator().manual_seed(n)
    src = torch.randint(0, 256, (n,), dtype=torch.uint8, generator=g).to(dev)
    dst = torch.zeros(n + 64, dtype=torch.uint8, device=dev)
    primitive.copy128(src, dst[:n])
    torch.cuda.synchronize()
    assert torch.equal(dst[:n], src) and int(dst[n:].sum()) == 0


@pytest.mark.parametrize("n", [0, 15, 16, 1000, (1 << 20) + 5, (64 << 20) + 16])
def test_read_xor_matches_numpy(dev, n):
    """The read-only yardstick really reads everything: its XOR of all whole
    16-byte vectors equals numpy's."""
    from mintccl_amd import primitive
    g = torch.Generator().manual_seed(77 + n)
    host = torch.randint(0, 256, (n,), dtype=torch.uint8, generator=g)
    got = primitive.read_xor(host.to(dev)).cpu().numpy().view(np.uint32)
    whole = host.numpy()[: n // 16 * 16].view(np.uint32).reshape(-1, 4)
    want = np.bitwise_xor.reduce(whole, axis=0) if len(whole) else np.zeros(4, np.uint32)
    assert got.tolist() == want.tolist()


@pytest.mark.parametrize("layout", [ll128.LAYOUT_PAIR, ll128.LAYOUT_WAVE64])
@pytest.mark.parametrize("n", SIZES)
def test_pack_unpack_match_oracle(dev, layout, n):
    from mintccl_amd import protocol
    raw = np.random.default_rng(n).integers(0, 256, n, dtype=np.uint8)
    d_raw = dev_bytes(raw, dev)
    base = 3 + n
    want = ll128.pack(raw, base, layout)
    msg = torch.full((want.size + 256,), 0xEE, dtype=torch.uint8, device=dev)
    protocol.pack(d_raw, base, layout, out=msg)
    torch.cuda.synchronize()
    got = msg.cpu().numpy()
    assert (got[:want.size] == want).all()
    assert (got[want.size:] == 0xEE).all()            # nothing written past the end
    out = torch.full((n + 64,), 0xEE, dtype=torch.uint8, device=dev)
    bad = torch.zeros(1, dtype=torch.int64, device=dev)
    if n:
        protocol.unpack(msg, out[:n], base, layout, bad_flags=bad)
    torch.cuda.synchronize()
    assert (out.cpu().numpy()[:n] == raw).all() and (out.cpu().numpy()[n:] == 0xEE).all()
    assert bad.item() == 0


@pytest.mark.parametrize("layout", [ll128.LAYOUT_PAIR, ll128.LAYOUT_WAVE64])
def test_unpack_counts_wrong_flags(dev, layout):
    from mintccl_amd import protocol
    raw = np.arange(20000, dtype=np.uint8)
    msg = ll128.pack(raw, 1, layout)
    msg[5 * 128 + (121 if layout == ll128.LAYOUT_PAIR else 61)] ^= 4
    msg[17 * 128 + 127] ^= 1
    d_msg = dev_bytes(msg, dev)
    out = torch.zeros(raw.size, dtype=torch.uint8, device=dev)
    bad = torch.zeros(1, dtype=torch.int64, device=dev)
    protocol.unpack(d_msg, out, 1, layout, bad_flags=bad)
    torch.cuda.synchronize()
    assert bad.item() == 2 == ll128.unpack(msg, raw.size, 1, layout)[1]


@pytest.mark.parametrize("layout", [ll128.LAYOUT_PAIR, ll128.LAYOUT_WAVE64])
@pytest.mark.parametrize("stride", [1, 0])
def test_config1_roundtrip_on_device(dev, layout, stride):
    # benchmark configuration 1 on the GPU: 1 MiB fp16 uniform[-1,1] seed 0
    from mintccl_amd import protocol
    x = uniform(524288, -1.0, 1.0, 0)
    d = x.to(dev)
    msg = protocol.pack(d, 1, layout, flag_stride=stride)
    want = ll128.pack(as_bytes(x), 1, layout, flag_stride=stride)
    assert (msg.cpu().numpy() == want).all()
    back = torch.empty_like(d)
    bad = torch.zeros(1, dtype=torch.int64, device=dev)
    protocol.unpack(msg, back, 1, layout, flag_stride=stride, bad_flags=bad)
    assert torch.equal(back.view(torch.int16), d.view(torch.int16)) and bad.item() == 0


@pytest.mark.parametrize("dt,tdt,bits", [("f16", torch.float16, 16), ("bf16", torch.bfloat16, 16),
                                         ("f32", torch.float32, 32)])
@pytest.mark.parametrize("n", [1, 7, 8, 100003, 1 << 20])
def test_elementwise_sum_random_bit_patterns(dev, dt, tdt, bits, n):
    from mintccl_amd import primitive
    a, b = random_bits(n, bits, n + 1), random_bits(n, bits, n + 2)
    iv, nv = (torch.int32, np.int32) if bits == 32 else (torch.int16, np.int16)
    ta = torch.from_numpy(a.view(nv)).to(dev).view(tdt)
    tb = torch.from_numpy(b.view(nv)).to(dev).view(tdt)
    got = primitive.Sum(ta, tb).view(iv).cpu().numpy()
    want = ring.add_rn(a, b, dt)
    assert ring.same_values(got, want, dt)
    if dt != "f16":       # bf16 canonicalises NaN, f32 NaNs aside: bits must agree
        w = want.view(np.uint16 if bits == 16 else np.uint32)
        g = got.view(np.uint16 if bits == 16 else np.uint32)
        nan = np.isnan(ring.to_float64(want, dt))
        assert (g[~nan] == w[~nan]).all()


def test_elementwise_sum_f16_special_values_and_subnormals(dev):
    from mintccl_amd import primitive
    sp = np.concatenate([special_values_f16(), np.arange(0, 1100, dtype=np.uint16),
                         np.arange(0x8000, 0x8000 + 1100, dtype=np.uint16)])
    aa, bb = np.meshgrid(sp, sp)
    aa, bb = aa.reshape(-1).copy(), bb.reshape(-1).copy()
    ta = torch.from_numpy(aa.view(np.int16)).to(dev).view(torch.float16)
    tb = torch.from_numpy(bb.view(np.int16)).to(dev).view(torch.float16)
    got = primitive.SumFP16(ta, tb).view(torch.int16).cpu().numpy()
    want = ring.add_rn(aa, bb, "f16")
    assert ring.same_values(got, want, "f16")
    finite = ~np.isnan(ring.to_float64(want, "f16"))
    assert (got.view(np.uint16)[finite] == want.view(np.uint16)[finite]).all()   # -0, subnormals


def test_alignment_is_rejected_not_faulted(lib, dev):
    from mintccl_amd import _lib
    buf = torch.zeros(4096, dtype=torch.uint8, device=dev)
    p = buf.data_ptr()
    assert lib.mint_copy_simple(p + 1, p + 2048, 64, 0, 0, 0) == _lib.ERR_ALIGN
    assert lib.mint_ll128_pack(p + 8, p + 2048, 64, 1, 1, 0, 0) == _lib.ERR_ALIGN
    assert lib.mint_ll128_pack(p, p + 2048, 64, 1, 1, 5, 0) == _lib.ERR_ARG
    assert lib.mint_elementwise_sum(p, p + 4, p + 2048, 8, 0, 0) == _lib.ERR_ALIGN


@pytest.mark.parametrize("via_lds", [0, 8])
def test_step_mix_moves_what_it_says(dev, via_lds):
    """The access-mix yardstick: with own-row loads and stores selected, the
    slot a wave stores into in its last step holds that step's own block in
    the lane order of the raw side (lane l, l % 4 != 3, carries the aligned
    16-byte vector l - l // 4 of the block).  The same with the own rows
    loaded straight into LDS (bit 8)."""
    from mintccl_amd import primitive
    waves, iters = 37, 5
    # f16 values in [1, 2): the store carries own + 0, which keeps such bits as they are
    rows = (torch.rand(waves * iters * 480, device=dev) + 1).to(torch.float16).view(torch.uint8)
    staging = torch.zeros(waves * 2048, dtype=torch.uint8, device=dev)
    primitive.step_mix(rows, staging, waves, iters, what=1 | 4 | via_lds)
    torch.cuda.synchronize()
    r, s = rows.cpu().numpy(), staging.cpu().numpy()
    for w in (0, 1, 17, waves - 1):
        block = r[((iters - 1) * waves + w) * 960:][:960]
        slot = s[w * 2048 + (iters & 1) * 1024:][:1024]
        for lane in range(64):
            if lane % 4 != 3:
                vec = lane - lane // 4
                assert (slot[lane * 16: lane * 16 + 16] == block[vec * 16: vec * 16 + 16]).all()
    # all three at once only has to run; loads alone leave staging as it is
    before = staging.clone()
    primitive.step_mix(rows, staging, waves, iters, what=1 | 2 | via_lds)
    torch.cuda.synchronize()
    assert torch.equal(staging, before)
    primitive.step_mix(rows, staging, waves, iters, what=7 | via_lds)
    torch.cuda.synchronize()


def test_step_mix_with_scalar_instructions_moves_the_same(dev):
    """what = 7 + 256 k: the scalar additions between the loads and the store
    of a step change nothing that is stored; a k without a kernel is refused."""
    from mintccl_amd import _lib, primitive
    waves, iters = 29, 6
    rows = (torch.rand(waves * iters * 480, device=dev) + 1).to(torch.float16).view(torch.uint8)
    plain = torch.zeros(waves * 2048, dtype=torch.uint8, device=dev)
    primitive.step_mix(rows, plain, waves, iters, what=7)
    for k in (2, 6, 12):
        busy = torch.zeros_like(plain)
        primitive.step_mix(rows, busy, waves, iters, what=7 + 256 * k)
        torch.cuda.synchronize()
        assert torch.equal(busy, plain)
    with pytest.raises(_lib.MintError):
        primitive.step_mix(rows, plain, waves, iters, what=7 + 256 * 3)
    with pytest.raises(_lib.MintError):
        primitive.step_mix(rows, plain, waves, iters, what=5 + 256 * 2)


def test_step_mix_saves_what_it_loads_from_staging(dev):
    """Bit 16: the block a wave took out of its staging slot goes back to HBM in
    the raw layout (lane l, l % 4 != 3: 16 bytes at vector l - l // 4; a flag
    lane: its 12 payload bytes behind the 48 vectors)."""
    from mintccl_amd import primitive
    waves, iters = 21, 4
    rows = torch.zeros(waves * iters * 960, dtype=torch.uint8, device=dev)
    staging = (torch.rand(waves * 1024, device=dev) + 1).to(torch.float16).view(torch.uint8)
    before = staging.clone()
    primitive.step_mix(rows, staging, waves, iters, what=2 | 16)
    torch.cuda.synchronize()
    assert torch.equal(staging, before)
    r, s = rows.cpu().numpy(), staging.cpu().numpy()
    for w in (0, 5, waves - 1):
        for i in (0, iters - 1):
            block = r[(i * waves + w) * 960:][:960]
            slot = s[w * 2048 + (i & 1) * 1024:][:1024]
            for lane in range(64):
                if lane % 4 != 3:
                    vec = lane - lane // 4
                    assert (block[vec * 16: vec * 16 + 16] == slot[lane * 16: lane * 16 + 16]).all()
                else:
                    at = 768 + 12 * (lane // 4)
                    assert (block[at: at + 12] == slot[lane * 16: lane * 16 + 12]).all()
    primitive.step_mix(rows, staging, waves, iters, what=2 | 4 | 16)       # only has to run
    torch.cuda.synchronize()

