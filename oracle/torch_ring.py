"""The ring reduce-scatter through the wire format, in PyTorch on the CPU.
Test infrastructure, never shipped: it is the CPU baseline that ``bench.py``
times beside the GPU kernel, and ``tests/test_oracle_ring`` checks it bit for
bit against the numpy restatement (``oracle.ring.reducescatter_wire``).

Same semantics as there (``7_reducescatter.py:54-73``, ``protocol.py:57-156``):
chunk ``c`` starts as rank ``c``'s own row; every hop packs the running value
into LL128 blocks of the wave64 layout (960 raw bytes -> 1024 message bytes, a
32-bit tag in the last 4 bytes of every 64-byte sector), the next rank in ring
order checks the tags, unpacks and adds its own row with one rounding
(``own + received``); after the last hop rank ``c`` stores the sum in its row
``c``.  Vectorised tensor operations only, so that torch's thread pool does
the work; float16 / bfloat16 / float32 addition on the CPU rounds once to
nearest even, which is what the numpy restatement pins.
"""
from __future__ import annotations

import torch

TORCH_DT = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}
BLOCK_RAW, BLOCK_MSG, SECTORS = 960, 1024, 16


def _pack(raw: torch.Tensor, flag_base: int) -> torch.Tensor:
    """uint8[n] -> uint8[ceil(n / 960) * 1024]; line L carries flag_base + L."""
    n = raw.numel()
    nblocks = -(-n // BLOCK_RAW)
    padded = torch.zeros(nblocks * BLOCK_RAW, dtype=torch.uint8)
    padded[:n] = raw
    blocks = padded.view(nblocks, BLOCK_RAW)
    msg = torch.empty(nblocks, SECTORS, 64, dtype=torch.uint8)
    msg[:, :, :48] = blocks[:, :768].reshape(nblocks, SECTORS, 48)
    msg[:, :, 48:60] = blocks[:, 768:].reshape(nblocks, SECTORS, 12)
    # sector i of block b belongs to line 8 b + i // 2
    lines = torch.arange(nblocks * SECTORS, dtype=torch.int64) // 2 + flag_base
    msg.view(-1, 64)[:, 60:64] = lines.to(torch.int32).view(torch.uint8).view(-1, 4)   # low 32 bits
    return msg.view(-1)


def _unpack(msg: torch.Tensor, nbytes: int, flag_base: int) -> torch.Tensor:
    nblocks = msg.numel() // BLOCK_MSG
    m = msg.view(nblocks, SECTORS, 64)
    lines = (torch.arange(nblocks * SECTORS, dtype=torch.int64) // 2 + flag_base) & 0xFFFFFFFF
    got = m.reshape(-1, 64)[:, 60:64].contiguous().view(torch.int32).view(-1).to(torch.int64) & 0xFFFFFFFF
    if not torch.equal(got, lines):
        raise AssertionError("a line arrived with a wrong tag")
    raw = torch.empty(nblocks, BLOCK_RAW, dtype=torch.uint8)
    raw[:, :768] = m[:, :, :48].reshape(nblocks, 768)
    raw[:, 768:] = m[:, :, 48:60].reshape(nblocks, 192)
    return raw.view(-1)[:nbytes]


def reducescatter_wire(bufs: list, dtype: str, ring: list | None = None, flag_base: int = 1) -> list:
    """bufs[r]: rank r's (world, n) tensor of `dtype`.  Returns the buffers after
    the call (new tensors)."""
    world = len(bufs)
    ring = ring or list(range(world)) + [0]
    cyc = ring[:-1]
    dt = TORCH_DT[dtype]
    out = [b.clone() for b in bufs]
    for c in range(world):
        i = cyc.index(c)
        order = cyc[i:] + cyc[:i]
        acc = bufs[order[0]][c].contiguous()
        nbytes = acc.numel() * acc.element_size()
        for r in order[1:]:
            received = _unpack(_pack(acc.view(torch.uint8), flag_base), nbytes, flag_base).view(dt)
            acc = bufs[r][c] + received                      # own + received, one rounding
        out[c][c] = _unpack(_pack(acc.view(torch.uint8), flag_base), nbytes, flag_base).view(dt)
    return out
