"""LL128 geometry and the stand-alone line codec.

Mirrors the constants of ``protocol.py:42-52``; the device functions of that
file (``load/save/recv/send/comp/wait/post_ll128``) live in
``csrc/protocol.hpp`` and ``csrc/ring.hpp``.  ``pack`` / ``unpack`` run the
codec kernels on device tensors through the C ABI.
"""
from __future__ import annotations

import torch

from . import _lib
from .common import VECTORIZED_BYTES, WARP_SIZE

PAYLOAD_WORK_THREAD = 16      # protocol.py:42
PAYLOAD_FLAG_THREAD = 8       # protocol.py:43
WORKGROUP_SIZE = 8            # protocol.py:44 lanes per line
ITERS_PER_SEND = 2            # protocol.py:45 (pair layout)
BYTES_LL128_MSG = 128         # protocol.py:47
BYTES_LL128_RAW = 120         # protocol.py:48
LINES_PER_WAVE = WARP_SIZE // WORKGROUP_SIZE                 # 8
BYTES_BLOCK_MSG = LINES_PER_WAVE * BYTES_LL128_MSG           # 1024
BYTES_BLOCK_RAW = LINES_PER_WAVE * BYTES_LL128_RAW           # 960
LAYOUT_PAIR, LAYOUT_WAVE64 = _lib.LAYOUT_PAIR, _lib.LAYOUT_WAVE64
assert PAYLOAD_WORK_THREAD == VECTORIZED_BYTES


def packed_bytes(nbytes: int, layout: int = LAYOUT_WAVE64) -> int:
    return _lib.lib().mint_ll128_packed_bytes(nbytes, layout)


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def pack(raw: torch.Tensor, flag_base: int = 1, layout: int = LAYOUT_WAVE64,
         flag_stride: int = 1, out: torch.Tensor | None = None) -> torch.Tensor:
    """Device tensor (any dtype, contiguous) -> uint8 tensor of LL128 lines."""
    if not raw.is_cuda or not raw.is_contiguous():
        raise ValueError("pack needs a contiguous device tensor")
    nbytes = raw.numel() * raw.element_size()
    need = packed_bytes(nbytes, layout)
    if out is None:
        out = torch.empty(need, dtype=torch.uint8, device=raw.device)
    elif out.numel() * out.element_size() < need:
        raise ValueError("output too small")
    with torch.cuda.device(raw.device):
        _lib.check(_lib.lib().mint_ll128_pack(raw.data_ptr(), out.data_ptr(), nbytes, flag_base,
                                              flag_stride, layout, _stream(raw)), "mint_ll128_pack")
    return out


def unpack(msg: torch.Tensor, out: torch.Tensor, flag_base: int = 1,
           layout: int = LAYOUT_WAVE64, flag_stride: int = 1,
           bad_flags: torch.Tensor | None = None) -> torch.Tensor:
    """LL128 lines -> ``out`` (its byte size says how much to unpack).
    ``bad_flags`` (int64[1], device) counts lines with an unexpected flag."""
    if not msg.is_cuda or not out.is_cuda or not out.is_contiguous():
        raise ValueError("unpack needs contiguous device tensors")
    nbytes = out.numel() * out.element_size()
    if msg.numel() * msg.element_size() < packed_bytes(nbytes, layout):
        raise ValueError("message too small")
    with torch.cuda.device(out.device):
        _lib.check(_lib.lib().mint_ll128_unpack(
            msg.data_ptr(), out.data_ptr(), nbytes, flag_base, flag_stride, layout,
            bad_flags.data_ptr() if bad_flags is not None else 0, _stream(out)),
            "mint_ll128_unpack")
    return out
