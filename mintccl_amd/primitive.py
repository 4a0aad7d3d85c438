"""Host handles on the device primitives.

The reference's ``primitive.py`` holds PTX device functions; their CDNA4
counterparts are in ``csrc/primitive.hpp``.  What can be called from the host
is exposed here so each primitive can be tested by itself: the 128-bit
load/store pair as a copy (``load128``/``store128``, ``primitive.py:180-203``)
and the reduce operator (``SumFP16``, ``primitive.py:232-247``) for f16, bf16
and f32.
"""
from __future__ import annotations

import torch

from . import _lib
from .common import DTYPE_CODE


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def copy128(src: torch.Tensor, dst: torch.Tensor, blocks: int = 0, threads: int = 0) -> None:
    """dst <- src with 16-byte loads / stores per lane."""
    n = src.numel() * src.element_size()
    if n != dst.numel() * dst.element_size():
        raise ValueError("size mismatch")
    with torch.cuda.device(src.device):
        _lib.check(_lib.lib().mint_copy_simple(src.data_ptr(), dst.data_ptr(), n, blocks, threads,
                                               _stream(src)), "mint_copy_simple")


def read_xor(src: torch.Tensor, out: torch.Tensor | None = None, blocks: int = 0,
             threads: int = 0) -> torch.Tensor:
    """XOR of all whole 16-byte vectors of ``src`` as four uint32 words (a
    read-only pass: the HBM read-bandwidth yardstick).  ``out`` (int32[4],
    zeroed by the caller) is XORed into; without it a fresh one is made."""
    n = src.numel() * src.element_size()
    if out is None:
        out = torch.zeros(4, dtype=torch.int32, device=src.device)
    with torch.cuda.device(src.device):
        _lib.check(_lib.lib().mint_read_xor(src.data_ptr(), n, out.data_ptr(), blocks, threads,
                                            _stream(src)), "mint_read_xor")
    return out


def step_mix(rows: torch.Tensor | None, staging: torch.Tensor | None, waves: int, iters: int,
             what: int = 7, sink: torch.Tensor | None = None) -> None:
    """The memory accesses of ``waves`` x ``iters`` ring steps with no ring around
    them (``what``: 1 own-row loads from ``rows``, 2 loads from ``staging``,
    4 stores into ``staging``, 8 with 1: own rows loaded straight into LDS
    instead of into registers, 16 without 1: the block is stored back into
    ``rows``; 256 * k with 7: k x 16 scalar additions per step between the
    loads and the store): the yardstick for what the device can do with
    the ring kernels' mix of accesses."""
    ref = rows if rows is not None else staging
    if sink is None and not what & 20:
        sink = torch.zeros(1, dtype=torch.int32, device=ref.device)
    nb = lambda t: 0 if t is None else t.numel() * t.element_size()
    ptr = lambda t: None if t is None else t.data_ptr()
    with torch.cuda.device(ref.device):
        _lib.check(_lib.lib().mint_step_mix(ptr(rows), nb(rows), ptr(staging), nb(staging), waves,
                                            iters, what, ptr(sink), _stream(ref)), "mint_step_mix")


def step_mix_deep(rows: torch.Tensor | None, staging: torch.Tensor | None, waves: int, iters: int,
                  what: int = 7, ahead: int = 1, partner: bool = True,
                  sink: torch.Tensor | None = None) -> None:
    """``step_mix`` with the loads ``ahead`` (1..3) steps ahead of their use and
    the stores never waited for: ``ahead + 1`` steps in flight per wavefront.
    ``staging`` holds ``waves * (ahead + 2)`` KiB; ``iters`` is a multiple of
    ``ahead + 1``; with ``partner`` a wavefront loads the lines another compute
    unit of its XCD stores."""
    ref = rows if rows is not None else staging
    if sink is None and not what & 4:
        sink = torch.zeros(1, dtype=torch.int32, device=ref.device)
    nb = lambda t: 0 if t is None else t.numel() * t.element_size()
    ptr = lambda t: None if t is None else t.data_ptr()
    with torch.cuda.device(ref.device):
        _lib.check(_lib.lib().mint_step_mix_deep(ptr(rows), nb(rows), ptr(staging), nb(staging),
                                                 waves, iters, what, ahead, int(partner), ptr(sink),
                                                 _stream(ref)), "mint_step_mix_deep")


def Sum(a: torch.Tensor, b: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """Elementwise ``rn(a + b)``, one rounding, by the ring kernels' own adder."""
    if a.dtype not in DTYPE_CODE or a.dtype != b.dtype or a.numel() != b.numel():
        raise ValueError("Sum needs two f16 / bf16 / f32 tensors of one shape")
    if out is None:
        out = torch.empty_like(a)
    with torch.cuda.device(a.device):
        _lib.check(_lib.lib().mint_elementwise_sum(a.data_ptr(), b.data_ptr(), out.data_ptr(),
                                                   a.numel(), DTYPE_CODE[a.dtype], _stream(a)),
                   "mint_elementwise_sum")
    return out


def SumFP16(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    if a.dtype != torch.float16:
        raise ValueError("SumFP16 takes float16 tensors")
    return Sum(a, b)


def xcd_map(blocks: int, device="cuda:0") -> torch.Tensor:
    """XCD each of ``blocks`` consecutive thread blocks lands on."""
    out = torch.empty(blocks, dtype=torch.int32, device=device)
    with torch.cuda.device(out.device):
        _lib.check(_lib.lib().mint_xcd_map(blocks, out.data_ptr(), _stream(out)), "mint_xcd_map")
    return out
