"""ctypes loader for ``liboracle_c.so`` (the C restatement).  Test
infrastructure, never shipped."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_DIR, "liboracle_c.so")
_lib = None

DT = {"f16": 0, "bf16": 1, "f32": 2}


def build(force: bool = False) -> str:
    if force or not os.path.exists(_SO) or (
            os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_DIR, "ll128_ref.c"))):
        subprocess.check_call(["make", "-C", _DIR, "-B", "liboracle_c.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        vp, sz, u64, ci = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint64, ctypes.c_int
        L.ref_line_count.restype = sz
        L.ref_line_count.argtypes = [sz, ci]
        L.ref_pack.restype = None
        L.ref_pack.argtypes = [vp, sz, u64, u64, ci, vp]
        L.ref_unpack.restype = sz
        L.ref_unpack.argtypes = [vp, sz, u64, u64, ci, vp]
        L.ref_add.restype = None
        L.ref_add.argtypes = [vp, vp, vp, sz, ci]
        L.ref_reducescatter_wire.restype = sz
        L.ref_reducescatter_wire.argtypes = [ctypes.POINTER(vp), ci, sz, ci,
                                             ctypes.POINTER(ci), ctypes.c_uint32, ci]
        _lib = L
    return _lib


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def pack(raw, flag_base=1, layout=0, flag_stride=1) -> np.ndarray:
    raw = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
    L = lib()
    msg = np.zeros(L.ref_line_count(raw.size, layout) * 128, dtype=np.uint8)
    L.ref_pack(_p(raw), raw.size, flag_base, flag_stride, layout, _p(msg))
    return msg


def unpack(msg, nbytes, flag_base=1, layout=0, flag_stride=1):
    msg = np.ascontiguousarray(msg).view(np.uint8).reshape(-1)
    raw = np.zeros(nbytes, dtype=np.uint8)
    bad = lib().ref_unpack(_p(msg), nbytes, flag_base, flag_stride, layout, _p(raw))
    return raw, int(bad)


def add(a, b, dtype: str) -> np.ndarray:
    a = np.ascontiguousarray(a).view(np.uint8).reshape(-1)
    b = np.ascontiguousarray(b).view(np.uint8).reshape(-1)
    out = np.empty_like(a)
    item = 4 if dtype == "f32" else 2
    lib().ref_add(_p(a), _p(b), _p(out), a.size // item, DT[dtype])
    return out


def reducescatter_wire(bufs: list, dtype: str, ring=None, epoch: int = 1, threads: int = 0) -> int:
    """In-place ring reduce-scatter on ``bufs`` (one contiguous uint8 array of
    ``world`` rows per rank), walked through the wire format.  Returns the
    number of messages with wrong tags (0)."""
    world = len(bufs)
    ring = list(ring) if ring is not None else list(range(world)) + [0]
    ptrs = (ctypes.c_void_p * world)(*[b.ctypes.data for b in bufs])
    cring = (ctypes.c_int * len(ring))(*ring)
    row = bufs[0].size // world
    return int(lib().ref_reducescatter_wire(ptrs, world, row, DT[dtype], cring, epoch, threads))
