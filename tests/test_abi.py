"""The C-ABI library loads without a GPU, exports every symbol the header
declares, agrees with the ctypes mirror on the descriptor layout, and its host
side validation (no kernel launch involved) returns the documented errors."""
import ctypes
import os
import re
import subprocess
import sys

import pytest

from mintccl_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mintccl.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mint_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    names = declared_functions()
    assert len(names) >= 12
    L = _lib.lib()
    for n in names:
        assert hasattr(L, n), f"{n} not exported by libmintccl.so"
        assert n in _lib.SYMBOLS, f"{n} has no ctypes signature"
    assert set(_lib.SYMBOLS) == set(names)


def test_version_and_strerror():
    L = _lib.lib()
    assert L.mint_version() == _lib.VERSION == 102
    assert L.mint_build_flags() == 0          # the in-tree library is a product build
    assert _lib.build_flags() == []
    assert L.mint_strerror(0) == b"ok"
    for code in range(-8, 0):
        assert L.mint_strerror(code) not in (b"ok", b"unknown error")
    assert L.mint_strerror(-99) == b"unknown error"


def test_descriptor_layout_matches_the_header(tmp_path):
    fields = [f for f, _ in _lib.RingOp._fields_]
    src = tmp_path / "layout.c"
    lines = ["#include <stdio.h>", "#include <stddef.h>", f'#include "{HEADER}"',
             "int main(void){", '  printf("%zu\\n", sizeof(mint_ring_op));']
    for f in fields:
        lines.append(f'  printf("%zu\\n", offsetof(mint_ring_op, {f}));')
    lines += ["  return 0;", "}"]
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-std=c11", "-o", str(exe), str(src)])
    out = [int(x) for x in subprocess.check_output([str(exe)]).split()]
    assert out[0] == ctypes.sizeof(_lib.RingOp)
    for f, off in zip(fields, out[1:]):
        assert getattr(_lib.RingOp, f).offset == off, f


def test_debug_struct_layout_matches_the_header(tmp_path):
    src = tmp_path / "layout.c"
    fields = [f for f, _ in _lib.RingDebug._fields_]
    lines = ["#include <stdio.h>", "#include <stddef.h>", f'#include "{HEADER}"',
             "int main(void){", '  printf("%zu\\n", sizeof(mint_ring_debug));']
    lines += [f'  printf("%zu\\n", offsetof(mint_ring_debug, {f}));' for f in fields]
    lines += ["  return 0;", "}"]
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-std=c11", "-o", str(exe), str(src)])
    out = [int(x) for x in subprocess.check_output([str(exe)]).split()]
    assert out[0] == ctypes.sizeof(_lib.RingDebug)
    for f, off in zip(fields, out[1:]):
        assert getattr(_lib.RingDebug, f).offset == off, f


def test_packed_bytes():
    L = _lib.lib()
    assert L.mint_ll128_packed_bytes(0, 0) == 0
    assert L.mint_ll128_packed_bytes(120, 0) == 128
    assert L.mint_ll128_packed_bytes(121, 0) == 256
    assert L.mint_ll128_packed_bytes(1 << 20, 0) == 8739 * 128
    assert L.mint_ll128_packed_bytes(1, 1) == 1024
    assert L.mint_ll128_packed_bytes(960, 1) == 1024
    assert L.mint_ll128_packed_bytes(961, 1) == 2048


def make_op(**kw):
    d = _lib.RingOp()
    d.op, d.protocol, d.dtype, d.world = _lib.OP_REDUCESCATTER, _lib.PROTO_LL128, _lib.F16, 8
    for i in range(9):
        d.ring[i] = i % 8
    for r in range(8):
        d.input[r] = d.output[r] = 0x10000000 + r * 0x1000000
        d.staging[r] = 0x70000000 + r * 0x1000000
    d.count_bytes, d.row_stride = 1 << 20, 1 << 20
    d.slot_bytes, d.nslots = 512 << 10, 8
    d.waves_per_channel_group, d.threads_per_block = 16, 256
    d.flag_epoch, d.status = 1, 0x60000000
    for k, v in kw.items():
        setattr(d, k, v)
    return d


def test_plan_geometry_without_a_gpu():
    L = _lib.lib()
    d = make_op()
    # 8 pipelines x 9 positions x (16 waves / 4 per block)
    assert L.mint_ring_grid_blocks(d) == 8 * 9 * 4
    assert L.mint_ring_staging_bytes(d) == (4 << 20) + 8 * 16 * 256 + _lib.TICKET_BYTES
    assert L.mint_ring_staging_bytes(make_op(credit_offset=8 << 20)) == (8 << 20) + 8 * 16 * 256 + _lib.TICKET_BYTES
    assert L.mint_ring_grid_blocks(make_op(op=_lib.OP_ALLGATHER, dtype=_lib.BYTES)) == 8 * 8 * 4
    d = make_op(op=_lib.OP_BROADCAST, dtype=_lib.BYTES, waves_per_channel_group=128, root=3)
    assert L.mint_ring_grid_blocks(d) == 8 * 32
    d = make_op(op=_lib.OP_REDUCE, waves_per_channel_group=128, root=3)
    assert L.mint_ring_grid_blocks(d) == 9 * 32
    # allreduce: 8 pipelines x 15 positions, two phases share a slot
    d = make_op(op=_lib.OP_ALLREDUCE, waves_per_channel_group=16, count_bytes=8 << 20)
    assert L.mint_ring_grid_blocks(d) == 8 * 15 * 4
    assert L.mint_ring_staging_bytes(d) == (4 << 20) + 8 * 2 * 16 * 256 + _lib.TICKET_BYTES
    # alltoall: 64 pipelines x 2 positions; a slot has one share per source rank
    d = make_op(op=_lib.OP_ALLTOALL, dtype=_lib.BYTES, waves_per_channel_group=16)
    for r in range(8):
        d.output[r] = 0x40000000 + r * 0x1000000
    assert L.mint_ring_grid_blocks(d) == 64 * 2 * 4
    assert L.mint_ring_staging_bytes(d) == (4 << 20) + 8 * 16 * 256 + _lib.TICKET_BYTES
    d.output[5] = d.input[2] + (3 << 20)                    # an output inside an input
    assert L.mint_ring_grid_blocks(d) == _lib.ERR_ARG
    assert L.mint_ring_grid_blocks(make_op(op=_lib.OP_ALLREDUCE, waves_per_channel_group=64)) \
        == _lib.ERR_GEOMETRY          # 512 KiB slot / 16 shares = 32 blocks per step


@pytest.mark.parametrize("kw,err", [
    (dict(world=0), _lib.ERR_ARG), (dict(world=9), _lib.ERR_ARG),
    (dict(op=12), _lib.ERR_ARG), (dict(protocol=2), _lib.ERR_ARG),
    (dict(op=_lib.OP_HYPERCUBE_REDUCESCATTER, protocol=_lib.PROTO_SIMPLE, slot_bytes=448 << 10,
          waves_per_channel_group=64), _lib.ERR_ARG),    # the hypercube kernels speak LL128 only
    (dict(op=_lib.OP_HYPERCUBE_ALLGATHER, dtype=_lib.BYTES, world=6, slot_bytes=320 << 10,
          waves_per_channel_group=64), _lib.ERR_ARG),    # 2^d corners
    (dict(op=_lib.OP_HYPERCUBE_REDUCESCATTER, dtype=_lib.BYTES, slot_bytes=448 << 10,
          waves_per_channel_group=64), _lib.ERR_ARG),    # a reduction needs a real dtype
    (dict(op=_lib.OP_ALLGATHER_TEMPORAL, dtype=_lib.BYTES, protocol=_lib.PROTO_SIMPLE,
          waves_per_channel_group=128), _lib.ERR_ARG),   # LL128 only
    (dict(op=_lib.OP_TREE_REDUCE, protocol=_lib.PROTO_SIMPLE, waves_per_channel_group=128),
     _lib.ERR_ARG),                                      # the tree kernels speak LL128 only
    (dict(op=_lib.OP_TREE_REDUCE, dtype=_lib.BYTES, waves_per_channel_group=128), _lib.ERR_ARG),
    (dict(dtype=_lib.BYTES), _lib.ERR_ARG),          # a reduction needs a real dtype
    (dict(flag_epoch=0), _lib.ERR_ARG), (dict(flag_epoch=4096), _lib.ERR_ARG),
    (dict(status=0), _lib.ERR_ARG), (dict(cache_policy=3), _lib.ERR_ARG),
    (dict(cache_policy=2, placement=0), _lib.ERR_ARG),   # XCD-local staging needs the local placement
    (dict(credit_offset=4096), _lib.ERR_GEOMETRY),       # inside the slots
    (dict(credit_offset=(4 << 20) + 100), _lib.ERR_GEOMETRY),
    (dict(row_fetch=2), _lib.ERR_ARG),
    (dict(op=_lib.OP_BROADCAST, dtype=_lib.BYTES, placement=1, waves_per_channel_group=16),
     _lib.ERR_GEOMETRY),                                 # 4 channels cannot be dealt to 8 XCDs
    (dict(flag_epoch=0, epoch_ptr=0x50000002), _lib.ERR_ALIGN),   # epoch word in device memory
    (dict(threads_per_block=100), _lib.ERR_ARG),
    (dict(slot_bytes=(512 << 10) + 512), _lib.ERR_GEOMETRY),
    (dict(slot_bytes=4096), _lib.ERR_GEOMETRY),        # less than one block per pipeline
    (dict(waves_per_channel_group=7), _lib.ERR_GEOMETRY),
    (dict(nslots=0), _lib.ERR_GEOMETRY),
    (dict(row_stride=1 << 19), _lib.ERR_ARG),         # rows would overlap
    (dict(total_bytes=(8 << 20) + 16), _lib.ERR_ARG), # more than world rows hold
    (dict(total_bytes=1001), _lib.ERR_ARG),           # not whole elements
    (dict(op=_lib.OP_REDUCE, total_bytes=4096), _lib.ERR_ARG),     # only for rows of one buffer
    (dict(op=_lib.OP_ALLREDUCE, waves_per_channel_group=16, total_bytes=4096), _lib.ERR_ARG),
    (dict(count_bytes=(1 << 20) + 1, row_stride=1 << 21), _lib.ERR_ARG),
    (dict(slot_bytes=1 << 30, nslots=8), _lib.ERR_TOO_LARGE),
    (dict(origin_cus=32), _lib.ERR_ARG), (dict(reserved1=1), _lib.ERR_ARG),
])
def test_plan_rejects_bad_descriptors(kw, err):
    assert _lib.lib().mint_ring_grid_blocks(make_op(**kw)) == err


def test_compute_units_set_apart_for_origins_grow_the_grid():
    """origin_cus: the blocks of an XCD are taken in rounds of 32; in every
    round so many take an origin, the others the receiving positions; the grid
    is whole rounds.  Only large ring broadcasts / allgathers under the local
    placement (and sendrecvs); ignored elsewhere."""
    L = _lib.lib()
    big = dict(op=_lib.OP_ALLGATHER, dtype=_lib.BYTES, placement=1, cache_policy=2,
               slot_bytes=512 << 10, nslots=3, waves_per_channel_group=64)
    assert L.mint_ring_grid_blocks(make_op(**big)) == 8 * 8 * 16                   # 4 rounds
    # 16 channels per XCD: 16 origins over 9 CUs (2 rounds), 112 receivers over 23 (5 rounds)
    assert L.mint_ring_grid_blocks(make_op(origin_cus=9, **big)) == 8 * 32 * 5
    assert L.mint_ring_grid_blocks(make_op(origin_cus=4, **big)) == 8 * 32 * 4     # the natural share
    assert L.mint_ring_grid_blocks(make_op(origin_cus=16, **big)) == 8 * 32 * 7
    bc = dict(op=_lib.OP_BROADCAST, dtype=_lib.BYTES, placement=1, cache_policy=2, count_bytes=64 << 20,
              slot_bytes=512 << 10, nslots=3, waves_per_channel_group=512)
    assert L.mint_ring_grid_blocks(make_op(origin_cus=9, **bc)) == 8 * 32 * 5
    # ignored: launches of fewer than 16 steps (their seats are taken in the order of
    # arrival), small grids, the spread placement, other collectives
    assert L.mint_ring_grid_blocks(make_op(origin_cus=9, **dict(bc, count_bytes=4 << 20))) == 8 * 8 * 16
    assert L.mint_ring_grid_blocks(make_op(origin_cus=9, **dict(bc, count_bytes=8 << 20))) == 8 * 32 * 5
    small = dict(big, waves_per_channel_group=16, slot_bytes=128 << 10)
    assert L.mint_ring_grid_blocks(make_op(origin_cus=9, **small)) == 8 * 8 * 4
    assert L.mint_ring_grid_blocks(make_op(origin_cus=9, **dict(big, placement=0, cache_policy=0))) == 8 * 8 * 16
    assert L.mint_ring_grid_blocks(make_op(origin_cus=9, placement=1, waves_per_channel_group=64)) == 8 * 9 * 16
    # a sendrecv over one hop: 64 channels per XCD, 20 CUs for the origins (4 rounds), 12 for
    # the destinations (6 rounds)
    sr = make_op(origin_cus=20, op=_lib.OP_SENDRECV, dtype=_lib.BYTES, placement=1, cache_policy=2,
                 count_bytes=256 << 20, route_len=2, slot_bytes=1536 << 10, nslots=4,
                 waves_per_channel_group=1536)
    sr.ring[0], sr.ring[1] = 0, 1
    assert L.mint_ring_grid_blocks(sr) == 8 * 32 * 4
    sr.threads_per_block = 128
    assert L.mint_ring_grid_blocks(sr) == 8 * 32 * 8


def test_plan_rejects_bad_buffers_and_rings():
    L = _lib.lib()
    d = make_op()
    d.input[3] = 0
    assert L.mint_ring_grid_blocks(d) == _lib.ERR_ARG
    d = make_op()
    d.staging[2] += 8
    assert L.mint_ring_grid_blocks(d) == _lib.ERR_ALIGN
    assert L.mint_ring_grid_blocks(make_op(flag_epoch=0, epoch_ptr=0x50000000)) > 0
    d = make_op(row_stride=(1 << 20) + 2)            # caller rows may start at any byte
    d.input[1] += 1
    d.output[1] += 1
    assert L.mint_ring_grid_blocks(d) > 0
    d = make_op()
    d.ring[8] = 1                                    # ring does not close
    assert L.mint_ring_grid_blocks(d) == _lib.ERR_ARG
    d = make_op()
    d.ring[3] = 2                                    # rank 2 twice
    assert L.mint_ring_grid_blocks(d) == _lib.ERR_ARG


def test_tree_plans_without_a_gpu():
    """Broadcast / reduce over a binary tree: one position per node; a reducing
    node's slot holds a share per child, with a credit word each."""
    L = _lib.lib()
    d = make_op(op=_lib.OP_TREE_BROADCAST, dtype=_lib.BYTES, waves_per_channel_group=128, root=3)
    assert L.mint_ring_grid_blocks(d) == 8 * 32
    assert L.mint_ring_staging_bytes(d) == (4 << 20) + 128 * 256 + _lib.TICKET_BYTES
    d = make_op(op=_lib.OP_TREE_REDUCE, waves_per_channel_group=128, root=3)
    assert L.mint_ring_grid_blocks(d) == 8 * 32
    assert L.mint_ring_staging_bytes(d) == (4 << 20) + 2 * 128 * 256 + _lib.TICKET_BYTES
    # 512 KiB slot / 2 shares = 256 blocks per step
    assert L.mint_ring_grid_blocks(make_op(op=_lib.OP_TREE_REDUCE, waves_per_channel_group=512)) \
        == _lib.ERR_GEOMETRY
    # buffers: root 3 heads the node order 3, 4, 5, 6, 7, 0, 1, 2; nodes 4..7 of it
    # (ranks 7, 0, 1, 2) are leaves and receive nothing in a reduce
    d = make_op(op=_lib.OP_TREE_REDUCE, waves_per_channel_group=128, root=3)
    for leaf in (7, 0, 1, 2):
        d.staging[leaf] = 0
    for r in range(8):
        if r != 3:
            d.output[r] = 0
    assert L.mint_ring_grid_blocks(d) == 8 * 32
    d.staging[4] = 0                                 # node 1 has children
    assert L.mint_ring_grid_blocks(d) == _lib.ERR_ARG
    d = make_op(op=_lib.OP_TREE_BROADCAST, dtype=_lib.BYTES, waves_per_channel_group=128, root=3)
    d.staging[3] = 0                                 # the root of a broadcast receives nothing
    for r in range(8):
        if r != 3:
            d.input[r] = 0
    d.output[3] = 0
    assert L.mint_ring_grid_blocks(d) == 8 * 32
    d.output[5] = 0
    assert L.mint_ring_grid_blocks(d) == _lib.ERR_ARG
    # the schedule listing covers the ring walks only
    n = ctypes.c_uint32(0)
    d = make_op(op=_lib.OP_TREE_REDUCE, waves_per_channel_group=128)
    assert L.mint_ring_schedule(d, 0, 0, 0, 0, None, None, None, None, ctypes.byref(n)) == _lib.ERR_ARG


def test_temporal_allgather_plan_without_a_gpu():
    """6_allgather.py:25-77: one pipeline of `world` positions that moves the rows
    one after the other; a slot holds one row's share."""
    L = _lib.lib()
    d = make_op(op=_lib.OP_ALLGATHER_TEMPORAL, dtype=_lib.BYTES, waves_per_channel_group=128)
    assert L.mint_ring_grid_blocks(d) == 8 * 32
    assert L.mint_ring_staging_bytes(d) == (4 << 20) + 128 * 256 + _lib.TICKET_BYTES
    # the same slot takes 8 x 64 blocks of the spatial schedule or 512 of this one
    assert L.mint_ring_grid_blocks(make_op(op=_lib.OP_ALLGATHER_TEMPORAL, dtype=_lib.BYTES,
                                           waves_per_channel_group=512)) == 8 * 128
    assert L.mint_ring_grid_blocks(make_op(op=_lib.OP_ALLGATHER, dtype=_lib.BYTES,
                                           waves_per_channel_group=512)) == _lib.ERR_GEOMETRY
    d.staging[5] = 0
    assert L.mint_ring_grid_blocks(d) == _lib.ERR_ARG
    # steps are numbered through all rows: 8 x 2^17 of them do not fit the 20-bit tag field
    d = make_op(op=_lib.OP_ALLGATHER_TEMPORAL, dtype=_lib.BYTES, waves_per_channel_group=1,
                slot_bytes=1024, count_bytes=960 << 17, row_stride=960 << 17)
    assert L.mint_ring_grid_blocks(d) == _lib.ERR_TOO_LARGE
    d = make_op(op=_lib.OP_ALLGATHER, dtype=_lib.BYTES, waves_per_channel_group=1,
                slot_bytes=8192, count_bytes=960 << 17, row_stride=960 << 17)
    assert L.mint_ring_grid_blocks(d) > 0


def test_launch_refuses_undersized_staging_before_touching_the_gpu():
    # The credit words lie behind the slots: a caller that allocates only
    # nslots * slot_bytes (the reference's recvbuff, 7_reducescatter.py:93)
    # is turned away instead of being written out of bounds.  The check comes
    # before any HIP call, so it runs without a GPU.
    L = _lib.lib()
    d = make_op()
    need = L.mint_ring_staging_bytes(d)
    assert need == (4 << 20) + 8 * 16 * 256 + _lib.TICKET_BYTES
    for have in (0, 4 << 20, need - 1):
        d.staging_bytes = have
        assert L.mint_ring_launch(d, None) == _lib.ERR_STAGING
    # a library built without wait accounting refuses a stats address
    d.staging_bytes = need
    dbg = _lib.RingDebug(0, 0, 0x1000)
    assert L.mint_ring_launch_debug(d, dbg, None) == _lib.ERR_ARG


def test_build_refuses_kernels_that_use_scratch():
    """The build reads hipcc's kernel-resource-usage remarks: a kernel whose
    locals were left in scratch memory computes the right bytes several times
    slower, so it is reported by name."""
    remarks = """\
a.hpp:9:1: remark: Function Name: _ZN4mint11ring_kernelILi0ELi3ELi2ELi1EEEvNS_8RingArgsE [-Rpass-analysis=kernel-resource-usage]
a.hpp:9:1: remark:     VGPRs: 91 [-Rpass-analysis=kernel-resource-usage]
a.hpp:9:1: remark:     ScratchSize [bytes/lane]: 2832 [-Rpass-analysis=kernel-resource-usage]
a.hpp:9:1: remark: Function Name: _ZN4mint11tree_kernelILi0ELi2EEEvNS_8RingArgsE [-Rpass-analysis=kernel-resource-usage]
a.hpp:9:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]
"""
    bad = _lib.kernels_with_scratch(remarks)
    assert bad == ["_ZN4mint11ring_kernelILi0ELi3ELi2ELi1EEEvNS_8RingArgsE (2832 bytes per lane)"]
    assert _lib.kernels_with_scratch("") == []
    assert "-Rpass-analysis=kernel-resource-usage" in _lib.HIPCC_FLAGS


def test_build_refuses_wide_stores_with_a_scalar_offset_register():
    """The build reads the device assembly: a 96- or 128-bit buffer store whose
    scalar offset operand is a register (not the constant 0) is reported; loads
    and narrower stores may use one."""
    asm = """\
\tbuffer_store_dwordx4 v[4:7], v41, s[20:23], s77 offen
\tbuffer_store_dwordx4 v[0:3], v42, s[20:23], 0 offen
\tbuffer_store_dwordx3 v[0:2], v42, s[20:23], s5 offen offset:16
\tbuffer_store_dwordx2 v[0:1], v42, s[20:23], s5 offen
\tbuffer_load_dwordx4 v[8:11], v28, s[24:27], s74 offen sc1
\tglobal_store_dwordx4 v[2:3], v[4:7], off nt
"""
    bad = _lib.stores_with_scalar_offset(asm)
    assert bad == ["buffer_store_dwordx4 v[4:7], v41, s[20:23], s77 offen",
                   "buffer_store_dwordx3 v[0:2], v42, s[20:23], s5 offen offset:16"]
    assert _lib.stores_with_scalar_offset("") == []


def test_missing_library_fails_loudly(tmp_path):
    code = ("import mintccl_amd._lib as l; l.SO_PATH=%r; l._lib=None\n"
            "try:\n    l.lib()\nexcept RuntimeError as e:\n    print('RAISED', 'no CPU fallback' in str(e))\n"
            % str(tmp_path / "nope.so"))
    out = subprocess.check_output([sys.executable, "-c", code], cwd=ROOT).decode()
    assert "RAISED True" in out


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "mintccl_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, f"{f} mentions the oracle"
