// LL128 line protocol for 64-lane wavefronts.
//
// Reference: protocol.py.  There an 8-lane "workgroup" moves two 128-byte
// lines per step (protocol.py:42-52) and lane 7 of each group carries 8
// payload bytes plus the 8-byte flag (load_ll128 :57-85, save_ll128 :87-100,
// recv_ll128 :102-130, send_ll128 :132-137, comp_ll128 :142-156).  That format
// rests on a 128-byte store becoming visible as a whole (protocol.py:31-35).
// On MI355X it does not: a consumer workgroup can see the second 64-byte
// sector of a line (the one with the flag) while the first still holds the
// previous occupant of the slot.  64-byte sectors were never seen torn.
//
// So the line keeps its 128 bytes, 120 of payload and 8 of flag, but the flag
// is a 32-bit tag stored once per 64-byte sector:
//     [0,60) payload | [60,64) tag | [64,124) payload | [124,128) tag
// and the unit is a *block*: one wavefront moves 8 lines (1 KiB of message,
// 960 payload bytes) with a single 16-byte access per lane.
//   lane l, l % 4 != 3 : aligned raw vector number  l - l / 4   (0..47)
//   lane l = 4 i + 3   : raw bytes [768 + 12 i, 780 + 12 i) and the tag of
//                        sector i
// Both sides are touched by contiguous accesses; the flag test is one 64-bit
// ballot.  A flag lane reads its 12 bytes with the same 16-byte load
// instruction as everybody else, starting 4 bytes early (the reference's own
// trick, protocol.py:74-82, widened to 64 lanes).
#pragma once
#include "primitive.hpp"

namespace mint {

// Caller rows may start at any byte: row accesses are typed with alignment 1
// (the device runs compute queues in unaligned access mode, and the compiler
// still emits one dwordx4 / dwordx3 / dwordx2 instruction per access).
typedef u32x4 u32x4_a1 __attribute__((aligned(1)));
typedef uint32_t u32x3 __attribute__((ext_vector_type(3)));
typedef u32x3 u32x3_a1 __attribute__((aligned(1)));
typedef u32x2 u32x2_a1 __attribute__((aligned(1)));

constexpr uint32_t kLineBytes = 128, kLinePayload = 120;
constexpr uint32_t kBlockMsg = 1024, kBlockRawLL = 960, kBlockRawSimple = 1024;
constexpr uint32_t kFlagLaneRaw = 768;    // first raw byte carried by a flag lane

// Per-lane constants of the wave64 layout.
struct LaneMap {
    uint32_t lane;
    uint32_t sector;     // 64-byte sector of the block this lane belongs to (0..15)
    bool flag_lane;
    uint32_t raw_off;    // first raw byte this lane carries, inside the block
    uint32_t raw_len;    // 16, or 12 on flag lanes
    __device__ __forceinline__ LaneMap() {
        lane = (uint32_t)lane_id();
        sector = lane >> 2;
        flag_lane = (lane & 3u) == 3u;
        raw_off = flag_lane ? kFlagLaneRaw + 12u * sector : (lane - sector) * 16u;
        raw_len = flag_lane ? 12u : 16u;
    }
};

// Byte-granular guarded access for the ragged end of a buffer: reads
// [off, off + len) clipped to nbytes, missing bytes read as zero.
__device__ __forceinline__ u32x4 load_guarded(const uint8_t* base_, uint64_t off, uint32_t len,
                                              uint64_t nbytes) {
    MINT_GLOBAL const uint8_t* base = as_global(base_);
    u32x4 v = {0u, 0u, 0u, 0u};
    if (off >= nbytes) return v;
    uint64_t have = nbytes - off;
    if (have >= len) {
        if (len == 16u) return *(MINT_GLOBAL const u32x4_a1*)(base + off);
        if (len == 12u) {
            u32x3 h = *(MINT_GLOBAL const u32x3_a1*)(base + off);
            v.x = h.x; v.y = h.y; v.z = h.z;
        } else {                                   // 8
            u32x2 h = *(MINT_GLOBAL const u32x2_a1*)(base + off);
            v.x = h.x; v.y = h.y;
        }
        return v;
    }
    uint32_t w[4] = {0u, 0u, 0u, 0u};
    for (uint32_t i = 0; i < (uint32_t)have; ++i)
        w[i >> 2] |= (uint32_t)base[off + i] << (8u * (i & 3u));
    v.x = w[0]; v.y = w[1]; v.z = w[2]; v.w = w[3];
    return v;
}
__device__ __forceinline__ void store_guarded(uint8_t* base_, uint64_t off, uint32_t len,
                                              uint64_t nbytes, u32x4 v) {
    MINT_GLOBAL uint8_t* base = as_global(base_);
    if (off >= nbytes) return;
    uint64_t have = nbytes - off;
    if (have >= len) {
        if (len == 16u) { *(MINT_GLOBAL u32x4_a1*)(base + off) = v; return; }
        if (len == 12u) {
            u32x3 h = {v.x, v.y, v.z};
            *(MINT_GLOBAL u32x3_a1*)(base + off) = h;
        } else {                                   // 8
            u32x2 h = {v.x, v.y};
            *(MINT_GLOBAL u32x2_a1*)(base + off) = h;
        }
        return;
    }
    uint32_t w[4] = {v.x, v.y, v.z, v.w};
    for (uint32_t i = 0; i < (uint32_t)have; ++i)
        base[off + i] = (uint8_t)(w[i >> 2] >> (8u * (i & 3u)));
}

// ---- wave64 LL128 block: raw side ----------------------------------------
// load_ll128 (protocol.py:57-85) in two halves, so that the load can be in
// flight while the wave does something else: ll_fetch_raw issues the load of
// raw block g of a row, ll_arrange (to be called where the value is first
// needed) puts the 12 payload bytes of a flag lane into .x/.y/.z; .w is
// don't-care there.  `full` (wave-uniform) says the block lies wholly inside
// the row; the ragged last block is read byte-guarded and arrives arranged.
__device__ __forceinline__ u32x4 ll_fetch_raw(const uint8_t* row, uint64_t row_bytes, uint32_t g,
                                              bool full, const LaneMap& m) {
    const uint64_t base = (uint64_t)g * kBlockRawLL;
    if (full) {
        // flag lanes start 4 bytes early so that all 64 lanes issue one
        // 16-byte load that stays inside the block
        const uint32_t off = m.flag_lane ? m.raw_off - 4u : m.raw_off;
#ifdef MINT_ROW_NOLOAD
        // diagnostic build: no load, the block's number instead of its bytes
        // (what a collective costs without its reads of the rows from HBM)
        return u32x4{g, off, 3u, 4u};
#else
        return __builtin_nontemporal_load(
            (MINT_GLOBAL const u32x4_a1*)(row + base + off));
#endif
    }
    return load_guarded(row, base + m.raw_off, m.raw_len, row_bytes);
}
__device__ __forceinline__ u32x4 ll_arrange(u32x4 v, bool full, const LaneMap& m) {
    if (full && m.flag_lane) { v.x = v.y; v.y = v.z; v.z = v.w; }
    return v;
}
__device__ __forceinline__ u32x4 ll_load_raw(const uint8_t* row, uint64_t row_bytes, uint32_t g,
                                             const LaneMap& m) {
    const bool full = (uint64_t)g * kBlockRawLL + kBlockRawLL <= row_bytes;    // wave-uniform
    return ll_arrange(ll_fetch_raw(row, row_bytes, g, full, m), full, m);
}
// save_ll128 (protocol.py:87-100): registers -> raw block g of a row.
__device__ __forceinline__ void ll_save_raw(uint8_t* row, uint64_t row_bytes, uint32_t g, bool full,
                                            const LaneMap& m, u32x4 v) {
    const uint64_t base = (uint64_t)g * kBlockRawLL;
    if (full) {
        if (!m.flag_lane) {
            __builtin_nontemporal_store(v, (MINT_GLOBAL u32x4_a1*)(row + base + m.raw_off));
        } else {
            u32x3 h = {v.x, v.y, v.z};
            __builtin_nontemporal_store(
                h, (MINT_GLOBAL u32x3_a1*)(row + base + m.raw_off));
        }
    } else {
        store_guarded(row, base + m.raw_off, m.raw_len, row_bytes, v);
    }
}
__device__ __forceinline__ void ll_save_raw(uint8_t* row, uint64_t row_bytes, uint32_t g,
                                            const LaneMap& m, u32x4 v) {
    const bool full = (uint64_t)g * kBlockRawLL + kBlockRawLL <= row_bytes;    // wave-uniform
    ll_save_raw(row, row_bytes, g, full, m, v);
}

// ---- wave64 LL128 block: message side ------------------------------------
// send_ll128 (protocol.py:132-137): one 1 KiB store, a tag riding in the
// last 4 bytes of every 64-byte sector.
template <int CP>
__device__ __forceinline__ void ll_send(const Window& dst, uint32_t off, u32x4 v, uint32_t tag,
                                        const LaneMap& m) {
    if (m.flag_lane) v.w = tag;
    st128<CP>(dst, off + m.lane * 16u, v);
}
// One poll of recv_ll128 (protocol.py:102-130): load the block, report whether
// all 16 sector tags are the expected one (64-lane ballot in place of any_sync).
template <int CP>
__device__ __forceinline__ bool ll_poll(const Window& src, uint32_t off, uint32_t tag,
                                        const LaneMap& m, u32x4& v) {
    v = ld128<CP>(src, off + m.lane * 16u);
    return wave_all(!m.flag_lane || v.w == tag);
}
// comp_ll128 (protocol.py:142-156): own + received; the tag word of a flag
// lane is not data - ll_send overwrites it - so all four words are added on
// every lane and no lane diverges.
template <int DT>
__device__ __forceinline__ u32x4 ll_comp(u32x4 own, u32x4 received) {
    return add_rn<DT>(own, received);
}

}  // namespace mint
