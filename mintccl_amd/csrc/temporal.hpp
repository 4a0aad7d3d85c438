// Allgather, temporal schedule: the whole grid works on one source rank's row
// at a time.
//
// Reference: allgather_kernel_temporal (6_allgather.py:25-77), the variant
// the reference's host function launches (6_allgather.py:157).  There every
// block walks the whole buffer in flag order, and who is the root of a line
// follows from the line number (`root_rank = flag // flags_per_rank`, :57):
// first everybody moves rank 0's chunk round the ring, then rank 1's, and so
// on.  (The ring kernels' per-source-rank pipelines are the *spatial* variant,
// :79-138; both leave the same bytes.)
//
// Here: one wavefront per (position, wave-channel).  The launch runs `world`
// phases; phase c is a broadcast of row c from rank c round the ring, and the
// wavefront of position h does in every phase what position h does - the
// origin loads, everybody else polls and keeps a copy, all but the last
// forward - on behalf of the rank that holds that position in the phase (the
// rank h places after rank c in ring order).  A wavefront thus keeps its role
// and changes its rank, which is what lets the origins sit on compute units
// of their own (origin_cus) although every rank is origin once.  Steps are
// numbered through the phases (phase c covers steps c * steps_per_row ...),
// so slots, sector tags and credit counts simply carry on from one phase to
// the next and a rank's staging holds one row's share, not `world`.  The link
// into rank c is idle during phase c; the origin of that phase still posts
// rank c's credit word for every step, so that the sender finds the slots
// free when the next phase starts.  A rank's credit word is posted by one
// wavefront per phase: before its first post in a phase a wavefront waits
// until the word has reached the phase's first step, i.e. until whoever
// served the rank before has finished (else an early post could release a
// slot the other has not emptied yet).  LL128 only.
#pragma once
#include "ring.hpp"

namespace mint {

template <int CPI>
__device__ __forceinline__ void temporal_walk(const RingArgs& a, const int h, const int w) {
    constexpr int LDCP = Policy<CPI>::LD, STCP = Policy<CPI>::ST;
    const LaneMap m;
    const int n = a.world;
    const uint32_t ring_bytes = a.nslots * a.slot_bytes;
    const uint32_t W = (uint32_t)a.waves, K = a.k_per_wave;
    const uint32_t chan = a.credit_off + (uint32_t)w * kCreditStride;
    const bool origin = h == 0, last = h == n - 1;
    const uint32_t epoch = launch_epoch(a);
    const uint64_t flag_hi = (uint64_t)epoch << 32;

    uint32_t gs = 0, slot = 0;                  // step counted through the phases, its slot
    for (int c = 0; c < n; ++c) {
        // whom this position works for in phase c
        const int i = ((int)a.start[c] + h) % n;
        const int rank = a.cyc[i], next = a.cyc[(i + 1) % n];
        const Window own(reinterpret_cast<const void*>(a.staging[rank]), ring_bytes);
        const Window nxt(reinterpret_cast<const void*>(a.staging[next]), ring_bytes);
        uint64_t* const own_tail = reinterpret_cast<uint64_t*>(a.staging[rank] + chan);
        const uint64_t* const nxt_tail = reinterpret_cast<const uint64_t*>(a.staging[next] + chan);
        uint32_t credits_seen = 0;              // (of `next`: another rank in every phase)
        // The rank's credit word is handed over from whoever posted it in the
        // phase before.  A receiving position posts from its first step on and
        // waits here; the origin, whose slot nobody writes in this phase, posts
        // once when the phase is over and waits there, so that it can load and
        // send while the phase before is still draining.
        const uint32_t base = gs;
        auto handed_over = [&]() __attribute__((always_inline)) -> bool {
            uint32_t seen = 0;
            return base == 0u || wait_count(own_tail, epoch, base, seen, a.spin_budget, a.status);
        };
        if (!origin && !handed_over()) {
            report_timeout(a.status, c, h, w, gs);
            return;
        }
        uint64_t row_bytes;
        uint32_t nblocks, nfull;
        row_extent(a, c, kBlockRawLL, row_bytes, nblocks, nfull);
        const uint8_t* in_row = reinterpret_cast<const uint8_t*>(a.input[rank]) +
                                (uint64_t)c * a.row_stride;
        uint8_t* out_row = reinterpret_cast<uint8_t*>(a.output[rank]) + (uint64_t)c * a.row_stride;
        uint32_t s = 0;
        if (origin && STCP == CP_NONE && K == 1u) {
            // The origin of this phase, one block per step, XCD-local staging:
            // rows fetched kAhead steps ahead, the credit read through the
            // scalar unit so that looking at it does not wait for the fetches
            // (a load from HBM takes 2.5 us under the ring's stores, and the
            // whole ring moves at the pace of the phase's origin).  Whole
            // blocks only; the ragged end of the row takes the loop below.
            constexpr uint32_t kAhead = 4;
            const uint32_t whole = nfull > (uint32_t)w ? (nfull - 1u - (uint32_t)w) / a.step_blocks + 1u : 0u;
            const uint32_t deep = whole < a.steps ? whole : a.steps;
            if (deep) {
                u32x4 vv[kAhead];
                auto fetch = [&](uint32_t of_step) __attribute__((always_inline)) {
                    uint32_t g = of_step * a.step_blocks + (uint32_t)w;
                    g = g < nfull ? g : nfull - 1u;          // beyond the whole blocks: any valid address
                    return ll_fetch_raw(in_row, row_bytes, g, true, m);
                };
                // (the prologue issues the queue a later step finds: a store
                // stands in for each step's send, to an unused part of the
                // credit line)
                uint64_t* const pad = const_cast<uint64_t*>(nxt_tail) + 8;
                vv[0] = fetch(0u);
#pragma unroll
                for (uint32_t d = 1; d < kAhead; ++d) {
                    compiler_fence();
                    st64_local(pad, 0ull);
                    compiler_fence();
                    vv[d] = fetch(d);
                }
                auto step = [&](auto phase) __attribute__((always_inline)) {
                    constexpr int B = decltype(phase)::value;
                    const uint32_t tag = (epoch << 20) | (gs + 1u);
                    const uint32_t need = gs >= a.nslots ? gs - a.nslots + 1 : 0;
                    for (uint32_t spins = 0; credits_seen < need; ++spins) {
                        const uint64_t cw = ld64_scalar(nxt_tail);
                        if ((uint32_t)(cw >> 32) == epoch && (uint32_t)cw >= need) {
                            credits_seen = (uint32_t)cw;
                            break;
                        }
                        if (spins >= a.spin_budget ||
                            ((spins & 63u) == 63u &&
                             __builtin_amdgcn_readfirstlane(ld32_agent_apart(a.status + 3)) != 0u)) {
                            report_timeout(a.status, c, h, w, gs);
                            __builtin_amdgcn_endpgm();
                        }
                        __builtin_amdgcn_s_sleep(1);
                    }
                    ll_send<STCP>(nxt, slot * a.slot_bytes + (uint32_t)w * kBlockMsg,
                                  ll_arrange(vv[B], true, m), tag, m);
                    compiler_fence();
                    vv[B] = fetch(s + kAhead);
                    slot = slot + 1 == a.nslots ? 0 : slot + 1;
                    ++s;
                    ++gs;
                };
                while (s < deep) {
                    step(std::integral_constant<int, 0>{});
                    if (s >= deep) break;
                    step(std::integral_constant<int, 1>{});
                    if (s >= deep) break;
                    step(std::integral_constant<int, 2>{});
                    if (s >= deep) break;
                    step(std::integral_constant<int, 3>{});
                }
            }
        }
        if (!origin && K == 1u) {
            // A receiving position, one block per step.  Vector-memory
            // operations of a wavefront retire in issue order, stores
            // included: in the plain loop below every poll waits for the
            // acknowledgement of the save (to HBM) and the send before it.
            // Here the credit word and the first poll of step s + 1 are issued
            // as soon as the tags of step s have been accepted, ahead of the
            // stores of step s, which then have a whole step to complete; the
            // credit for the slot is posted at that moment too (the block is
            // in registers).  Two register buffers, hence two copies of the
            // body; the prologue issues the queue a later step finds (stand-ins
            // for the stores go to an unused part of this wave-channel's
            // credit line); a wave that gives up ends on the spot.
            // Whole blocks only; the ragged end of the row takes the loop below.
            const uint32_t whole = nfull > (uint32_t)w ? (nfull - 1u - (uint32_t)w) / a.step_blocks + 1u : 0u;
            const uint32_t fast = whole < a.steps ? whole : a.steps;
            if (fast) {
                u32x4 rr[2];
                uint64_t cw[2] = {0, 0};
                uint64_t* const pad = own_tail + 8;
                auto store_pad = [&]() __attribute__((always_inline)) {
                    if (STCP == CP_NONE) st64_local(pad, 0ull);
                    else st64_agent(pad, 0ull);
                };
                auto give_up = [&]() __attribute__((always_inline)) {
                    report_timeout(a.status, c, h, w, gs);
                    __builtin_amdgcn_endpgm();
                };
                const uint32_t lane_off = (uint32_t)w * kBlockMsg + m.lane * 16u;
                if (!last) cw[0] = ld64_agent(nxt_tail);
                rr[0] = ld128<LDCP>(own, slot * a.slot_bytes + lane_off);
                compiler_fence();
                store_pad();                    // the post
                store_pad();                    // the save
                if (!last) store_pad();         // the send
                compiler_fence();
                auto step = [&](auto phase) __attribute__((always_inline)) {
                    constexpr int B = decltype(phase)::value, B1 = B ^ 1;
                    const uint32_t next_slot = slot + 1 == a.nslots ? 0 : slot + 1;
                    const uint32_t tag = (epoch << 20) | (gs + 1u);
                    const uint32_t need = gs >= a.nslots ? gs - a.nslots + 1 : 0;
                    const uint32_t at = slot * a.slot_bytes + (uint32_t)w * kBlockMsg;
                    if (!wave_all(!m.flag_lane || rr[B].w == tag)) {
                        for (uint32_t spins = 0;; ++spins) {
                            if (spins >= a.spin_budget || ((spins & 63u) == 63u && aborted(a.status)))
                                give_up();
                            __builtin_amdgcn_s_sleep(1);
                            compiler_fence();
                            if (ll_poll<LDCP>(own, at, tag, m, rr[B])) break;
                        }
                    }
                    if (!last) {
                        asm volatile("" : "+v"(cw[B]));
                        if (credits_seen < need) {
                            const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(cw[B] >> 32));
                            const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)cw[B]);
                            if (hi == epoch && lo >= need) credits_seen = lo;
                            else if (!wait_count(nxt_tail, epoch, need, credits_seen, a.spin_budget,
                                                 a.status))
                                give_up();
                        }
                    }
                    // the next step's credit word and first poll go out ahead of this step's stores
                    compiler_fence();
                    if (!last) cw[B1] = ld64_agent(nxt_tail);
                    rr[B1] = ld128<LDCP>(own, next_slot * a.slot_bytes + lane_off);
                    compiler_fence();
                    // post_ll128 (protocol.py:183-189); every lane stores the same word
                    if (STCP == CP_NONE) st64_local(own_tail, flag_hi | (uint64_t)(gs + 1));
                    else st64_agent(own_tail, flag_hi | (uint64_t)(gs + 1));
                    ll_save_raw(out_row, row_bytes, s * a.step_blocks + (uint32_t)w, true, m, rr[B]);
                    if (!last) ll_send<STCP>(nxt, at, rr[B], tag, m);
                    compiler_fence();
                    slot = next_slot;
                    ++s;
                    ++gs;
                };
                while (s < fast) {
                    step(std::integral_constant<int, 0>{});
                    if (s >= fast) break;
                    step(std::integral_constant<int, 1>{});
                }
            }
        }
        for (; s < a.steps; ++s, ++gs) {
            const uint32_t tag = (epoch << 20) | (gs + 1u);
            // wait_ll128 (protocol.py:161-180)
            const uint32_t need = gs >= a.nslots ? gs - a.nslots + 1 : 0;
            if (!last && !wait_count(nxt_tail, epoch, need, credits_seen, a.spin_budget, a.status)) {
                report_timeout(a.status, c, h, w, gs);
                return;
            }
            for (uint32_t k = 0; k < K; ++k) {
                const uint32_t idx = k * W + (uint32_t)w;
                const uint32_t g = s * a.step_blocks + idx;
                if (g >= nblocks) break;
                const uint32_t at = slot * a.slot_bytes + idx * kBlockMsg;
                u32x4 x;
                if (origin) {
                    // load_ll128 (6_allgather.py:61-62)
                    x = ll_load_raw(in_row, row_bytes, g, m);
                } else {
                    // recv_ll128 (:63-65), bounded
                    compiler_fence();
                    for (uint32_t spins = 0; !ll_poll<LDCP>(own, at, tag, m, x); ++spins) {
                        if (spins >= a.spin_budget ||
                            ((spins & 63u) == 63u && aborted(a.status))) {
                            report_timeout(a.status, c, h, w, gs);
                            return;
                        }
                        __builtin_amdgcn_s_sleep(1);
                        compiler_fence();
                    }
                    ll_save_raw(out_row, row_bytes, g, m, x);          // save_ll128 (:68-69)
                }
                if (!last) ll_send<STCP>(nxt, at, x, tag, m);          // send_ll128 (:72-73)
            }
            // post_ll128 (protocol.py:183-189)
            if (!origin && lane_id() == 0) {
                if (STCP == CP_NONE) st64_local(own_tail, flag_hi | (uint64_t)(gs + 1));
                else st64_agent(own_tail, flag_hi | (uint64_t)(gs + 1));
            }
            slot = slot + 1 == a.nslots ? 0 : slot + 1;
        }
        if (origin) {
            // the slots of the origin's rank stayed empty in this phase: all of its steps at once
            if (!handed_over()) {
                report_timeout(a.status, c, h, w, gs);
                return;
            }
            if (lane_id() == 0) {
                if (STCP == CP_NONE) st64_local(own_tail, flag_hi | (uint64_t)gs);
                else st64_agent(own_tail, flag_hi | (uint64_t)gs);
            }
        }
    }
}

// Seats are dealt as for the ring kernels.
template <int CPI>
__global__ void __launch_bounds__(512) temporal_kernel(const RingArgs a) {
    __shared__ int entry[1];
    const int wpb = (int)(blockDim.x >> 6);
    const int wib = (int)__builtin_amdgcn_readfirstlane((uint32_t)wave_in_block());
    const Seat st = take_seat(a, wpb, wib, wib, (MINT_LDS int*)entry);
    if (!st.ok) return;
    temporal_walk<CPI>(a, st.h, st.w);
}

}  // namespace mint
