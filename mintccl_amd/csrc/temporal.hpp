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
// Here: one wavefront per (rank, wave-channel).  The launch runs `world`
// phases; in phase c the rank at ring index i is position (i - index of c) of
// a broadcast of row c from rank c: the origin loads, everybody else polls
// and keeps a copy, all but the last forward.  Steps are numbered through the
// phases (phase c covers steps c * steps_per_row ...), so slots, sector tags
// and credit counts simply carry on from one phase to the next and a rank's
// staging holds one row's share, not `world`.  The link into rank c is idle
// during phase c; its receiver - the origin of that phase - still posts its
// credit word for every step, so that the sender finds the slots free when
// the next phase starts.  LL128 only.
#pragma once
#include "ring.hpp"

namespace mint {

enum : int { OP_ALLGATHER_TEMPORAL = 9 };

template <int CPI>
__device__ __forceinline__ void temporal_walk(const RingArgs& a, const int i, const int w) {
    constexpr int LDCP = Policy<CPI>::LD, STCP = Policy<CPI>::ST;
    const LaneMap m;
    const int n = a.world;
    const int rank = a.cyc[i], next = a.cyc[(i + 1) % n];
    const uint32_t ring_bytes = a.nslots * a.slot_bytes;
    const Window own(reinterpret_cast<const void*>(a.staging[rank]), ring_bytes);
    const Window nxt(reinterpret_cast<const void*>(a.staging[next]), ring_bytes);
    const uint32_t W = (uint32_t)a.waves, K = a.k_per_wave;
    const uint32_t chan = a.credit_off + (uint32_t)w * kCreditStride;
    uint64_t* const own_tail = reinterpret_cast<uint64_t*>(a.staging[rank] + chan);
    const uint64_t* const nxt_tail = reinterpret_cast<const uint64_t*>(a.staging[next] + chan);
    const uint32_t epoch =
        a.epoch_word ? __builtin_amdgcn_readfirstlane(__hip_atomic_load(
                           as_global(a.epoch_word), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
                     : a.epoch;
    const uint64_t flag_hi = (uint64_t)epoch << 32;
    uint32_t credits_seen = 0;

    uint32_t gs = 0, slot = 0;                  // step counted through the phases, its slot
    for (int c = 0; c < n; ++c) {
        const int h = (i - (int)a.start[c] + n) % n;
        const bool origin = h == 0, last = h == n - 1;
        uint64_t row_bytes;
        uint32_t nblocks, nfull;
        row_extent(a, c, kBlockRawLL, row_bytes, nblocks, nfull);
        const uint8_t* in_row = reinterpret_cast<const uint8_t*>(a.input[rank]) +
                                (uint64_t)c * a.row_stride;
        uint8_t* out_row = reinterpret_cast<uint8_t*>(a.output[rank]) + (uint64_t)c * a.row_stride;
        for (uint32_t s = 0; s < a.steps; ++s, ++gs) {
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
            // post_ll128 (protocol.py:183-189) - by the origin too, whose slot
            // nobody wrote in this phase
            if (lane_id() == 0) {
                if (STCP == CP_NONE) st64_local(own_tail, flag_hi | (uint64_t)(gs + 1));
                else st64_agent(own_tail, flag_hi | (uint64_t)(gs + 1));
            }
            slot = slot + 1 == a.nslots ? 0 : slot + 1;
        }
    }
}

// Seats are dealt as for the ring kernels (position = ring index of the rank).
template <int CPI>
__global__ void __launch_bounds__(512) temporal_kernel(const RingArgs a) {
    const int wpb = (int)(blockDim.x >> 6);
    const int wib = (int)__builtin_amdgcn_readfirstlane((uint32_t)wave_in_block());
    const Seat st = take_seat(a, wpb, wib);
    if (!st.ok) return;
    temporal_walk<CPI>(a, st.h, st.w);
}

}  // namespace mint
