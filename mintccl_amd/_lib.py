"""ctypes binding of ``libmintccl.so`` (C ABI declared in ``include/mintccl.h``).

The shared library is the product's only compute path: if it is missing the
import of any operator fails with an error that says how to build it.  There is
no CPU or PyTorch fallback.
"""
from __future__ import annotations

import ctypes
import os
import shutil
import subprocess

_PKG = os.path.dirname(os.path.abspath(__file__))
_ROOT = os.path.dirname(_PKG)
# MINTCCL_LIBRARY points at a diagnostic build (see build(defines=...)); it has
# to exist like the in-tree one.
SO_PATH = os.getenv("MINTCCL_LIBRARY") or os.path.join(_PKG, "libmintccl.so")
_CSRC = os.path.join(_PKG, "csrc")
SRC = os.path.join(_CSRC, "mintccl.hip")
FAMILY_SRC = os.path.join(_CSRC, "ring_family.hip")     # compiled once per element type
BUILD_DIR = os.path.join(_PKG, "_build")

MAX_RANKS = 8
STATUS_WORDS = 4
MAX_EPOCH = 4095          # sector tags carry a 12-bit launch epoch

(OK, ERR_ARG, ERR_ALIGN, ERR_GEOMETRY, ERR_RESIDENCY, ERR_HIP, ERR_TOO_LARGE,
 ERR_STAGING, ERR_NOT_READY) = 0, -1, -2, -3, -4, -5, -6, -7, -8
VERSION = 102             # the interface version this binding was written for
TICKET_BYTES = 20 * 1024  # the end of every rank's staging: room for the seat tickets
SEAT_STATE_WORDS = 17     # mint_ring_seat: counters of one XCD in a simulated launch
BUILD_RING_STATS, BUILD_ROW_NOLOAD = 1, 2
LAYOUT_PAIR, LAYOUT_WAVE64 = 0, 1
F16, BF16, F32, BYTES = 0, 1, 2, 3
PROTO_LL128, PROTO_SIMPLE = 0, 1
(OP_SENDRECV, OP_BROADCAST, OP_REDUCE, OP_ALLGATHER, OP_REDUCESCATTER, OP_ALLREDUCE,
 OP_ALLTOALL, OP_TREE_BROADCAST, OP_TREE_REDUCE, OP_ALLGATHER_TEMPORAL,
 OP_HYPERCUBE_REDUCESCATTER, OP_HYPERCUBE_ALLGATHER) = range(12)
PLACE_SPREAD, PLACE_LOCAL = 0, 1
FETCH_INLINE, FETCH_LDS = 0, 1

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed FP32 instructions are kept out of all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
    # the compiler reports every kernel's registers and scratch memory; build()
    # refuses a kernel that uses scratch (see there)
    "-Rpass-analysis=kernel-resource-usage",
]


class RingOp(ctypes.Structure):
    """``mint_ring_op`` of include/mintccl.h, field for field."""
    _fields_ = [
        ("op", ctypes.c_int32), ("protocol", ctypes.c_int32),
        ("dtype", ctypes.c_int32), ("world", ctypes.c_int32),
        ("ring", ctypes.c_int32 * (MAX_RANKS + 1)),
        ("route_len", ctypes.c_int32), ("root", ctypes.c_int32),
        ("input", ctypes.c_uint64 * MAX_RANKS),
        ("output", ctypes.c_uint64 * MAX_RANKS),
        ("staging", ctypes.c_uint64 * MAX_RANKS),
        ("staging_bytes", ctypes.c_uint64),
        ("count_bytes", ctypes.c_uint64), ("row_stride", ctypes.c_uint64),
        ("slot_bytes", ctypes.c_uint32), ("nslots", ctypes.c_uint32),
        ("waves_per_channel_group", ctypes.c_uint32),
        ("threads_per_block", ctypes.c_uint32),
        ("placement", ctypes.c_int32), ("cache_policy", ctypes.c_int32),
        ("flag_epoch", ctypes.c_uint32), ("spin_budget", ctypes.c_uint32),
        ("status", ctypes.c_uint64),
        ("row_fetch", ctypes.c_int32), ("credit_offset", ctypes.c_uint32),
        ("total_bytes", ctypes.c_uint64),
        ("epoch_ptr", ctypes.c_uint64),
        ("origin_cus", ctypes.c_uint32), ("reserved1", ctypes.c_uint32),
    ]


class RingDebug(ctypes.Structure):
    """``mint_ring_debug``: the test hooks of ``mint_ring_launch_debug``."""
    _fields_ = [("skip_origin", ctypes.c_uint32), ("reserved0", ctypes.c_uint32),
                ("stats", ctypes.c_uint64)]


# name -> (restype, argtypes); every symbol include/mintccl.h declares
_vp, _sz, _u64, _u32, _i = (ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint64,
                            ctypes.c_uint32, ctypes.c_int)
_ip = ctypes.POINTER(ctypes.c_int)
_u32p = ctypes.POINTER(ctypes.c_uint32)
_opp = ctypes.POINTER(RingOp)
_dbgp = ctypes.POINTER(RingDebug)
SYMBOLS = {
    "mint_version": (_i, []),
    "mint_build_flags": (_i, []),
    "mint_strerror": (ctypes.c_char_p, [_i]),
    "mint_device_info": (_i, [_ip, _ip, _ip]),
    "mint_xcd_map": (_i, [_i, _vp, _vp]),
    "mint_copy_simple": (_i, [_vp, _vp, _sz, _i, _i, _vp]),
    "mint_read_xor": (_i, [_vp, _sz, _vp, _i, _i, _vp]),
    "mint_step_mix": (_i, [_vp, _sz, _vp, _sz, _i, _i, _i, _vp, _vp]),
    "mint_step_mix_deep": (_i, [_vp, _sz, _vp, _sz, _i, _i, _i, _i, _i, _vp, _vp]),
    "mint_ll128_packed_bytes": (_sz, [_sz, _i]),
    "mint_ll128_pack": (_i, [_vp, _vp, _sz, _u64, _u64, _i, _vp]),
    "mint_ll128_unpack": (_i, [_vp, _vp, _sz, _u64, _u64, _i, _vp, _vp]),
    "mint_elementwise_sum": (_i, [_vp, _vp, _vp, _sz, _i, _vp]),
    "mint_ring_staging_bytes": (_sz, [_opp]),
    "mint_ring_grid_blocks": (_i, [_opp]),
    "mint_ring_schedule": (_i, [_opp, _i, _i, _i, _u32, _u32p, _u32p, _u32p, _u32p, _u32p]),
    "mint_ring_seat": (_i, [_opp, _i, _i, _i, ctypes.POINTER(ctypes.c_uint64), _ip, _ip, _ip]),
    "mint_ring_launch": (_i, [_opp, _vp]),
    "mint_ring_launch_debug": (_i, [_opp, _dbgp, _vp]),
    "mint_ring_launch_static": (_i, [_opp, _vp]),
    "mint_static_init": (_i, []),
    "mint_epoch_advance": (_i, [_vp, _vp, _sz, _i, _vp]),
    "mint_torn_line_probe": (_i, [_vp, _sz, _i, _i, _i, _i, _i, _u32, _u32, _vp, _vp]),
}

_lib = None


def kernels_with_scratch(remarks: str) -> list[str]:
    """Names of the kernels whose ``-Rpass-analysis=kernel-resource-usage``
    remarks report a non-zero scratch size."""
    import re
    out, name = [], "?"
    for line in remarks.splitlines():
        m = re.search(r"Function Name: (\S+)", line)
        if m:
            name = m.group(1)
        m = re.search(r"ScratchSize \[bytes/lane\]: (\d+)", line)
        if m and int(m.group(1)) > 0:
            out.append(f"{name} ({m.group(1)} bytes per lane)")
    return out


def stores_with_scalar_offset(asm: str) -> list[str]:
    """The 96- and 128-bit buffer stores of a device assembly listing whose
    scalar offset operand is a register.  Such a store was seen to pick up the
    next vector instruction's write to its first data register (the compiler
    leaves a wait state behind a wide store only when that operand is a
    constant), so the kernels keep a store's whole offset in the vector
    register and build() refuses a listing that holds one."""
    import re
    pat = re.compile(r"^\s*buffer_store_dwordx[34]\s+v\[\d+:\d+\],\s*(?:v\d+|off),\s*s\[\d+:\d+\],\s*(s\d+|m0|vcc_lo|vcc_hi)\b")
    return [line.strip() for line in asm.splitlines() if pat.match(line)]


def build(verbose: bool = False, defines: tuple[str, ...] = (), so_path: str | None = None) -> str:
    """Compile the HIP sources for gfx950 into ``libmintccl.so`` (in-tree).

    The ring kernels are one translation unit per element type; the five
    compilations run side by side and are linked at the end.  ``defines``
    (``-DMINT_RING_STATS``: wait accounting per ring position,
    ``-DMINT_ROW_NOLOAD``: whole blocks of own rows are not loaded - wrong
    results, for timing a collective without its HBM reads) and ``so_path``
    make a diagnostic build beside the product's; ``MINTCCL_LIBRARY`` loads it,
    ``mint_build_flags`` says which one is loaded."""
    out = so_path or os.path.join(_PKG, "libmintccl.so")
    build_dir = BUILD_DIR if so_path is None else out + ".objs"
    os.makedirs(build_dir, exist_ok=True)
    units = [(SRC, list(defines), os.path.join(build_dir, "mintccl.o"))]
    for dt in range(4):
        units.append((FAMILY_SRC, [f"-DMINT_FAMILY_DT={dt}", *defines],
                      os.path.join(build_dir, f"ring_family_{dt}.o")))
    procs = []
    for src, defs, obj in units:
        # every unit compiles in a directory of its own: the compiler leaves the
        # device assembly there (-save-temps), which is looked at below
        tmp = obj + ".tmp"
        shutil.rmtree(tmp, ignore_errors=True)
        os.makedirs(tmp)
        cmd = ["hipcc", *HIPCC_FLAGS, *defs, "-save-temps=obj", "-c", "-o",
               os.path.join(tmp, os.path.basename(obj)), src]
        if verbose:
            print(" ".join(cmd))
        procs.append((cmd, tmp, obj, subprocess.Popen(cmd, stdout=subprocess.PIPE,
                                                      stderr=subprocess.PIPE, text=True)))
    errors, spilling, hazards = [], [], []
    for cmd, tmp, obj, proc in procs:
        _, err = proc.communicate()
        if proc.returncode != 0:
            errors.append(f"{' '.join(cmd)}\n{err}")
        else:
            listings = [f for f in os.listdir(tmp) if f.endswith("gfx950.s")]
            if not listings:
                errors.append(f"{' '.join(cmd)}\nleft no device assembly in {tmp}")
            for f in listings:
                with open(os.path.join(tmp, f)) as fh:
                    hazards += [f"{os.path.basename(obj)}: {line}"
                                for line in stores_with_scalar_offset(fh.read())]
            os.replace(os.path.join(tmp, os.path.basename(obj)), obj)
        shutil.rmtree(tmp, ignore_errors=True)
        spilling += kernels_with_scratch(err)
    if errors:
        raise RuntimeError("hipcc failed:\n" + "\n".join(errors))
    if hazards:
        raise RuntimeError("wide buffer stores with their offset in a scalar register "
                           "(see stores_with_scalar_offset):\n" + "\n".join(hazards[:20]))
    if spilling:
        # A walk whose locals the optimiser could not keep in registers (it
        # happens when closures capture closures) still computes the right
        # bytes, five times slower: fail the build instead.
        raise RuntimeError("kernels that use scratch memory: " + ", ".join(spilling))
    link = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out,
            *[obj for _, _, obj in units]]
    if verbose:
        print(" ".join(link))
    proc = subprocess.run(link, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc link failed:\n{proc.stderr}")
    return out


class MintError(RuntimeError):
    def __init__(self, code: int, where: str):
        self.code = code
        msg = lib().mint_strerror(code).decode() if _lib is not None else str(code)
        super().__init__(f"{where}: {msg} ({code})")


def lib():
    """The loaded library.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(SO_PATH):
            raise RuntimeError(
                f"{SO_PATH} is missing: the HIP extension has not been built. "
                "Run `python -c 'import __graft_entry__ as g; g.build()'` "
                "(or mintccl_amd._lib.build()) in the repository root. "
                "There is no CPU fallback.")
        L = ctypes.CDLL(SO_PATH)
        # The descriptor below is laid out for one version of the interface: a
        # stale or diagnostic library of another version would read it shifted.
        L.mint_version.restype, L.mint_version.argtypes = ctypes.c_int, []
        if L.mint_version() != VERSION:
            raise RuntimeError(
                f"{SO_PATH} speaks interface version {L.mint_version()}, this binding {VERSION}: "
                "rebuild it (mintccl_amd._lib.build())")
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        # A library that was built to return wrong results (timing without the
        # reads of the rows) is only loaded by who asks for it by name.
        flags = L.mint_build_flags()
        if flags & BUILD_ROW_NOLOAD and os.getenv("MINTCCL_ALLOW_DIAGNOSTIC") != "1":
            raise RuntimeError(
                f"{SO_PATH} was built with -DMINT_ROW_NOLOAD and returns wrong results by design; "
                "set MINTCCL_ALLOW_DIAGNOSTIC=1 to load it for timing")
        _lib = L
    return _lib


def build_flags() -> list[str]:
    """Names of the diagnostic switches the loaded library was built with
    (empty for a product build)."""
    flags = lib().mint_build_flags()
    return [name for bit, name in ((BUILD_RING_STATS, "MINT_RING_STATS"),
                                   (BUILD_ROW_NOLOAD, "MINT_ROW_NOLOAD")) if flags & bit]


def check(code: int, where: str) -> None:
    if code != OK:
        raise MintError(code, where)
