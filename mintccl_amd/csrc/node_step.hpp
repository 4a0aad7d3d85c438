// Whole steps of a node that takes blocks from NIN senders and passes them on
// to NOUT receivers: what the walks of tree.hpp and hypercube.hpp do in a
// step, with the node's shape a compile-time constant and everything that does
// not change from step to step taken out of the loop.
//
// Reference: none (see tree.hpp and hypercube.hpp); the pieces are the
// reference's load / recv / comp / save / send of LL128 blocks
// (protocol.py:57-156) and its credit words (protocol.py:161-189).
//
// The order of a step is the order of the ring kernels' adding loop (ring.hpp,
// "whole steps of the adding collectives"), for the same reasons: the credit
// words of the receivers are asked for ahead of the polls and looked at after
// them; the polls of all senders go out together; the node's own row block of
// the following step is fetched behind the polls, so that the wait for the
// polls leaves exactly that fetch in flight (nothing behind the polls is issued
// conditionally, fetch addresses are clamped into the row); tags, credit posts, the
// additions, the farthest sender first, then the save or the sends.  UP: the
// node adds what it receives to its own block (reduce, reduce-scatter); else
// it passes on what it receives or, with no sender, its own block (broadcast,
// allgather).  One block per wave-channel and step, XCD-local staging, LL128.
#pragma once
#include "ring.hpp"

namespace mint {

constexpr int kNodeMaxEdges = 3;

// What a node's whole-step loop needs to know, all of it fixed for the launch.
struct NodeEdges {
    uint32_t in_off[kNodeMaxEdges];       // byte offset of sender j's share inside a slot of this rank
    uint32_t out_off[kNodeMaxEdges];      // ... of this node's share inside a slot of receiver j
    uint64_t* in_tail[kNodeMaxEdges];     // credit word this node posts for sender j
    const uint64_t* out_tail[kNodeMaxEdges];   // credit word receiver j posts for this node
};

// Runs steps 0 .. whole - 1 (each a whole block of this wave-channel) and
// returns; `credits_seen` carries on into the caller's loop.  Gives up like the
// other walks: the first wavefront whose bounded wait runs out reports it and
// ends.
template <int DT, int CPI, bool UP, int NIN, int NOUT>
__device__ __forceinline__ void node_whole_steps(const RingArgs& a, const int p, const int h, const int w,
                                                 const uint32_t whole, const Window& own,
                                                 const Window& out0, const Window& out1,
                                                 const Window& out2, const NodeEdges& e,
                                                 const uint8_t* in_row, uint8_t* out_row,
                                                 const uint64_t row_bytes, const uint32_t nfull,
                                                 uint32_t (&credits_seen)[kNodeMaxEdges]) {
    static_assert(CPI == 2, "XCD-local staging only");
    static_assert(NIN <= kNodeMaxEdges && NOUT <= kNodeMaxEdges && NIN + NOUT > 0, "a node's shape");
    constexpr int LDCP = Policy<CPI>::LD, STCP = Policy<CPI>::ST;
    constexpr bool LOAD = UP || NIN == 0;
    constexpr bool SAVE = UP ? NOUT == 0 : NIN != 0;
    constexpr uint64_t kDataLanes = 0x7777777777777777ull;    // every lane but the fourth of a sector
    const LaneMap m;
    const uint32_t epoch = launch_epoch(a);
    const uint64_t flag_hi = (uint64_t)epoch << 32;
    const uint32_t ring_bytes = a.nslots * a.slot_bytes;
    const uint32_t lane_off = (uint32_t)w * kBlockMsg + m.lane * 16u;
    const uint32_t last_full = nfull - 1u;

    uint32_t slot_off = 0;
    uint32_t tag = (epoch << 20) | 1u;
    int32_t need = 1 - (int32_t)a.nslots;            // credits the step needs, if positive
    uint32_t g0 = (uint32_t)w;
    u32x4 vv[2] = {u32x4{0u, 0u, 0u, 0u}, u32x4{0u, 0u, 0u, 0u}};
    uint64_t cw[kNodeMaxEdges] = {0, 0, 0};

    auto fetch = [&](uint32_t g) __attribute__((always_inline)) {
        g = g < last_full ? g : last_full;               // beyond the whole blocks: any valid address
        return ll_fetch_raw(in_row, row_bytes, g, true, m);
    };
    auto give_up = [&]() __attribute__((always_inline)) {
        report_timeout(a.status, p, h, w, (uint32_t)(need + (int32_t)a.nslots) - 1u);
        __builtin_amdgcn_endpgm();
    };
    auto step = [&](auto phase) __attribute__((always_inline)) {
        constexpr int B = decltype(phase)::value, B1 = B ^ 1;
        u32x4 r[kNodeMaxEdges];
        // wait_ll128 (protocol.py:161-180): the words of the receivers that have
        // not yet been seen far enough, asked for together
#pragma unroll
        for (int j = 0; j < NOUT; ++j)
            if ((int32_t)credits_seen[j] < need) cw[j] = ld64_agent(e.out_tail[j]);
        compiler_fence();
#pragma unroll
        for (int j = 0; j < NIN; ++j) r[j] = ld128<LDCP>(own, e.in_off[j] + lane_off, slot_off);
        compiler_fence();
        if (LOAD) vv[B1] = fetch(g0 + a.step_blocks);
        compiler_fence();
        if (NIN > 0) {
            // recv_ll128 (protocol.py:102-130)
            uint32_t pending = 0;
#pragma unroll
            for (int j = 0; j < NIN; ++j)
                if ((__ballot(r[j].w == tag) | kDataLanes) != ~0ull) pending |= 1u << j;
            for (uint32_t spins = 0; pending; ++spins) {
                if (spins >= a.spin_budget || ((spins & 63u) == 63u && aborted(a.status))) give_up();
                __builtin_amdgcn_s_sleep(1);
                compiler_fence();
#pragma unroll
                for (int j = 0; j < NIN; ++j) {
                    if (!(pending & (1u << j))) continue;
                    r[j] = ld128<LDCP>(own, e.in_off[j] + lane_off, slot_off);
                    if ((__ballot(r[j].w == tag) | kDataLanes) == ~0ull) pending &= ~(1u << j);
                }
            }
            // post_ll128 (protocol.py:183-189): the step is in registers, the
            // slot is free; every lane stores the same word
            const uint64_t posted = flag_hi | (uint64_t)(uint32_t)(need + (int32_t)a.nslots);
#pragma unroll
            for (int j = 0; j < NIN; ++j) st64_local(e.in_tail[j], posted);
        }
#pragma unroll
        for (int j = 0; j < NOUT; ++j) {
            asm volatile("" : "+v"(cw[j]));
            if ((int32_t)credits_seen[j] < need) {
                // (compared in vector registers: every lane holds the word)
                if (__ballot((uint32_t)(cw[j] >> 32) == epoch && (int32_t)(uint32_t)cw[j] >= need) != 0ull)
                    credits_seen[j] = __builtin_amdgcn_readfirstlane((uint32_t)cw[j]);
                else if (!wait_count(e.out_tail[j], epoch, (uint32_t)need, credits_seen[j],
                                     a.spin_budget, a.status))
                    give_up();
            }
        }
        u32x4 x = vv[B];
        if (LOAD) x = ll_arrange(x, true, m);
        // recv + comp (protocol.py:102-156): the farthest sender first
#pragma unroll
        for (int j = 0; j < NIN; ++j) {
            if constexpr (DT != DT_BYTES) {
                x = UP ? ll_comp<DT>(x, r[j]) : r[j];
            } else {
                x = r[j];
            }
        }
        if (SAVE) ll_save_raw(out_row, row_bytes, g0, true, m, x);
        if (NOUT > 0) {
            if (m.flag_lane) x.w = tag;
            const uint32_t at = lane_off + slot_off;
            st128<STCP>(out0, e.out_off[0] + at, x);
            if (NOUT > 1) st128<STCP>(out1, e.out_off[1] + at, x);
            if (NOUT > 2) st128<STCP>(out2, e.out_off[2] + at, x);
        }
        ++tag; ++need;
        g0 += a.step_blocks;
        slot_off += a.slot_bytes;
        slot_off = slot_off == ring_bytes ? 0u : slot_off;
    };
    // an odd number of steps starts with one step out of the second buffer, so
    // that the loop is whole pairs and has one way out
    const uint32_t end_tag = tag + whole;
    if (whole & 1u) {
        if (LOAD) vv[1] = fetch(g0);
        step(std::integral_constant<int, 1>{});
    } else if (LOAD) {
        vv[0] = fetch(g0);
    }
    while (tag != end_tag) {
        step(std::integral_constant<int, 0>{});
        step(std::integral_constant<int, 1>{});
    }
}

}  // namespace mint
