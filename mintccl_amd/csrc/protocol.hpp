// LL128 line protocol for 64-lane wavefronts.
//
// Reference: protocol.py.  There an 8-lane "workgroup" moves two 128-byte
// lines per step (protocol.py:42-52) and lane 7 of each group carries 8
// payload bytes plus the 8-byte flag (load_ll128 :57-85, save_ll128 :87-100,
// recv_ll128 :102-130, send_ll128 :132-137, comp_ll128 :142-156).
//
// Here the unit is a *block*: one wavefront moves 8 lines (1 KiB of message,
// 960 payload bytes) with a single 16-byte access per lane.
//   lane l, l % 8 != 7 : aligned raw vector number  l - l / 8   (0..55)
//   lane l = 8 j + 7   : raw bytes [896 + 8 j, 904 + 8 j) and the flag of line j
// so a block is 60 aligned 16-byte raw vectors, and both the raw side and the
// message side are touched by contiguous, 16-byte-aligned accesses; the flag
// test is one 64-bit ballot.  The flag lanes read their 8 bytes with the same
// 16-byte load as everybody else (vector 56 + j / 2, half j % 2): the
// reference's own trick (protocol.py:74-82) widened to 64 lanes.
#pragma once
#include "primitive.hpp"

namespace mint {

constexpr uint32_t kLineBytes = 128, kLinePayload = 120;
constexpr uint32_t kBlockMsg = 1024, kBlockRawLL = 960, kBlockRawSimple = 1024;

// Per-lane constants of the wave64 layout.
struct LaneMap {
    uint32_t lane;
    uint32_t line;       // line of the block this lane belongs to (0..7)
    bool flag_lane;
    uint32_t raw_off;    // first raw byte this lane carries, inside the block
    uint32_t raw_len;    // 16, or 8 on flag lanes
    uint32_t ld_off;     // aligned 16-byte vector the lane loads
    bool hi_half;        // flag lanes: which half of that vector is theirs
    __device__ __forceinline__ LaneMap() {
        lane = (uint32_t)lane_id();
        line = lane >> 3;
        flag_lane = (lane & 7u) == 7u;
        raw_off = flag_lane ? 896u + 8u * line : (lane - line) * 16u;
        raw_len = flag_lane ? 8u : 16u;
        ld_off = flag_lane ? (56u + (line >> 1)) * 16u : raw_off;
        hi_half = flag_lane && (line & 1u);
    }
};

// Byte-granular guarded access for the ragged end of a buffer: reads
// [off, off + len) clipped to nbytes, missing bytes read as zero.
__device__ __forceinline__ u32x4 load_guarded(const uint8_t* base, uint64_t off, uint32_t len,
                                              uint64_t nbytes) {
    u32x4 v = {0u, 0u, 0u, 0u};
    if (off >= nbytes) return v;
    uint64_t have = nbytes - off;
    if (have >= len) {
        if (len == 16u) return *reinterpret_cast<const u32x4*>(base + off);
        u32x2 h = *reinterpret_cast<const u32x2*>(base + off);
        v.x = h.x; v.y = h.y;
        return v;
    }
    uint32_t w[4] = {0u, 0u, 0u, 0u};
    for (uint32_t i = 0; i < (uint32_t)have; ++i)
        w[i >> 2] |= (uint32_t)base[off + i] << (8u * (i & 3u));
    v.x = w[0]; v.y = w[1]; v.z = w[2]; v.w = w[3];
    return v;
}
__device__ __forceinline__ void store_guarded(uint8_t* base, uint64_t off, uint32_t len,
                                              uint64_t nbytes, u32x4 v) {
    if (off >= nbytes) return;
    uint64_t have = nbytes - off;
    if (have >= len) {
        if (len == 16u) { *reinterpret_cast<u32x4*>(base + off) = v; return; }
        u32x2 h = {v.x, v.y};
        *reinterpret_cast<u32x2*>(base + off) = h;
        return;
    }
    uint32_t w[4] = {v.x, v.y, v.z, v.w};
    for (uint32_t i = 0; i < (uint32_t)have; ++i)
        base[off + i] = (uint8_t)(w[i >> 2] >> (8u * (i & 3u)));
}

// ---- wave64 LL128 block: raw side ----------------------------------------
// load_ll128 (protocol.py:57-85): raw block g of a row -> registers.  On
// flag lanes .x/.y hold the 8 payload bytes; .z/.w are don't-care.
__device__ __forceinline__ u32x4 ll_load_raw(const uint8_t* row, uint64_t row_bytes, uint32_t g,
                                             const LaneMap& m) {
    const uint64_t base = (uint64_t)g * kBlockRawLL;
    u32x4 v;
    if (base + kBlockRawLL <= row_bytes) {       // wave-uniform
        v = ld128_stream(row + base + m.ld_off);
        if (m.hi_half) { v.x = v.z; v.y = v.w; }
    } else {
        v = load_guarded(row, base + m.raw_off, m.raw_len, row_bytes);
    }
    return v;
}
// save_ll128 (protocol.py:87-100): registers -> raw block g of a row.
__device__ __forceinline__ void ll_save_raw(uint8_t* row, uint64_t row_bytes, uint32_t g,
                                            const LaneMap& m, u32x4 v) {
    const uint64_t base = (uint64_t)g * kBlockRawLL;
    if (base + kBlockRawLL <= row_bytes) {
        if (!m.flag_lane) {
            st128_stream(row + base + m.raw_off, v);
        } else {
            u32x2 h = {v.x, v.y};
            st64_stream(row + base + m.raw_off, h);
        }
    } else {
        store_guarded(row, base + m.raw_off, m.raw_len, row_bytes, v);
    }
}

// ---- wave64 LL128 block: message side ------------------------------------
// Flag of line j of a block whose first line carries `first`.
__device__ __forceinline__ uint64_t ll_line_flag(uint64_t first, uint64_t stride,
                                                 const LaneMap& m) {
    return first + (uint64_t)m.line * stride;
}
// send_ll128 (protocol.py:132-137): one 1 KiB store, flags riding in the
// last 8 bytes of every line.
template <int CP>
__device__ __forceinline__ void ll_send(const Window& dst, uint32_t off, u32x4 v, uint64_t flag,
                                        const LaneMap& m) {
    if (m.flag_lane) { v.z = (uint32_t)flag; v.w = (uint32_t)(flag >> 32); }
    st128<CP>(dst, off + m.lane * 16u, v);
}
// One poll of recv_ll128 (protocol.py:102-130): load the block, report whether
// all 8 flags are the expected ones (64-lane ballot in place of any_sync).
template <int CP>
__device__ __forceinline__ bool ll_poll(const Window& src, uint32_t off, uint64_t flag,
                                        const LaneMap& m, u32x4& v) {
    v = ld128<CP>(src, off + m.lane * 16u);
    const bool ok = !m.flag_lane || (v.z == (uint32_t)flag && v.w == (uint32_t)(flag >> 32));
    return wave_all(ok);
}
// comp_ll128 (protocol.py:142-156): own + received; the flag words of the
// flag lanes are not data - ll_send overwrites them - so all four words are
// added on every lane and no lane diverges.
template <int DT>
__device__ __forceinline__ u32x4 ll_comp(u32x4 own, u32x4 received) {
    return add_rn<DT>(own, received);
}

}  // namespace mint
