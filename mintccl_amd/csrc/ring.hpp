// Ring chunk scheduler and the fused ring-collective kernel.
//
// Reference: the scheduling arithmetic that lives inline in every kernel
// (2_sendrecv_indirect.py:61,76-77,93; 3_sendrecv_buffer.py:32-34,46-47,73-74;
// 6_allgather.py:91-102,137-138; 7_reducescatter.py:23-34,43-44,75-77) and the
// per-round credit handshake post_ll128 / wait_ll128 (protocol.py:161-189).
//
// One launch runs every virtual rank.  The work is a set of independent
// *pipelines* (one per reduced / gathered row; one in total for sendrecv,
// broadcast and reduce).  A pipeline visits `hops + 1` *positions*: position 0
// is the origin (loads raw data and sends), the last position is the sink
// (receives and saves), the ones in between receive, optionally add their own
// row or save a copy, and forward.  For reduce and reducescatter the root
// occupies both position 0 and the last position (the reference lets the root
// run both roles in one thread with a lag of `world_size` rounds,
// 5_reduce.py:79-89, 7_reducescatter.py:57-67; here they are different
// wavefronts, so nothing has to lag).
//
// Each (pipeline, position) is served by W *wave-channels*; wave-channel w of
// position h talks only to wave-channel w of positions h-1 and h+1.  Staging
// of a rank is `nslots` slots of `slot_bytes`; a slot holds one *step* of all
// pipelines, split evenly: step s of pipeline p lives at
//     (s % nslots) * slot_bytes + p * (slot_bytes / P)
// and inside it block i = k * W + w is wave-channel w's k-th block of the step.
// Every 64-byte sector of step s carries the 32-bit tag (epoch << 20 | s + 1):
// successive occupants of a slot differ in the step, launches differ in the
// epoch, so a slot is never cleared (the reference's idea of a unique,
// never-zero flag, 2_sendrecv_indirect.py:59-61); the caller clears staging
// when its 12-bit epoch counter wraps.  Flow control is a consumer-owned credit word per wave-channel
// ((epoch << 32) | steps consumed) that the upstream producer polls before it
// reuses a slot - separate from the data lines, unlike wait/post_ll128 which
// overload the flag word of slot 0.
#pragma once
#include "protocol.hpp"

namespace mint {

enum : int { OP_SENDRECV = 0, OP_BROADCAST = 1, OP_REDUCE = 2, OP_ALLGATHER = 3,
             OP_REDUCESCATTER = 4 };
enum : int { PROTO_LL128 = 0, PROTO_SIMPLE = 1 };
enum : int { PLACE_SPREAD = 0, PLACE_LOCAL = 1 };

constexpr int kMaxRanks = 8;
constexpr uint32_t kCreditStride = 256;   // per wave-channel: line 0 tail, line 1 head

struct RingArgs {
    int32_t op, world, pipes, hops;       // positions per pipeline = hops + 1
    int32_t waves;                        // W, wave-channels per (pipeline, position)
    int32_t blocks_per_group;             // thread blocks per (pipeline, position)
    int32_t placement;
    int32_t cyc_len;                      // ring length, or route length for sendrecv
    uint8_t cyc[kMaxRanks + 1];           // ring order / route
    uint8_t start[kMaxRanks];             // per pipeline: index of its root in cyc
    uint64_t input[kMaxRanks], output[kMaxRanks], staging[kMaxRanks];
    uint64_t row_bytes, row_stride;
    uint32_t nblocks;                     // blocks per row
    uint32_t steps;                       // steps per row
    uint32_t slot_bytes, nslots;
    uint32_t step_msg;                    // slot_bytes / pipes
    uint32_t step_blocks;                 // step_msg / 1024
    uint32_t k_per_wave;                  // step_blocks / waves
    uint32_t credit_off;                  // offset of the credit words in staging
    uint32_t epoch, spin_budget;
    uint64_t* status;
    uint32_t skip_origin;
};

struct Role {
    int rank, next;
    bool load, recv, reduce, save, send;
};

__device__ __forceinline__ Role role_of(const RingArgs& a, int p, int h) {
    Role r;
    const int s = a.start[p];
    r.rank = a.cyc[(s + h) % a.cyc_len];
    r.next = a.cyc[(s + h + 1) % a.cyc_len];
    const bool origin = h == 0, sink = h == a.hops;
    const bool reducing = a.op == OP_REDUCE || a.op == OP_REDUCESCATTER;
    const bool copying_all = a.op == OP_BROADCAST || a.op == OP_ALLGATHER;
    r.recv = !origin;
    r.send = !sink;
    r.load = origin || (reducing && !sink);
    r.reduce = reducing && !origin && !sink;
    r.save = sink || (copying_all && !origin);
    return r;
}

// First waiter that gives up records who it was; everybody else sees word 3.
__device__ __forceinline__ void report_timeout(uint64_t* status, int p, int h, int w,
                                               uint64_t step) {
    if (lane_id() == 0) {
        unsigned long long* s = reinterpret_cast<unsigned long long*>(status);
        if (atomicCAS(s, 0ull, 1ull) == 0ull) {
            st64_agent(status + 1, ((uint64_t)p << 32) | ((uint64_t)h << 16) | (uint64_t)w);
            st64_agent(status + 2, step);
        }
        st64_agent(status + 3, 1ull);
    }
}
__device__ __forceinline__ bool aborted(const uint64_t* status) {
    return __builtin_amdgcn_readfirstlane((uint32_t)ld64_agent(status + 3)) != 0u;
}

// Spin until the credit / head word at `word` carries this epoch and a count
// of at least `need`.  Returns false when the budget ran out or somebody
// aborted.  (wait_ll128, protocol.py:161-180, with a bound.)
__device__ __forceinline__ bool wait_count(const uint64_t* word, uint32_t epoch, uint32_t need,
                                           uint32_t& cached, uint32_t budget,
                                           const uint64_t* status, bool acquire) {
    if (cached >= need) return true;
    for (uint32_t spins = 0;; ++spins) {
        uint64_t v = acquire ? ld64_acquire(word) : ld64_agent(word);
        uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
        uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
        if (hi == epoch && lo >= need) { cached = lo; return true; }
        if (spins >= budget) return false;
        if ((spins & 63u) == 63u && aborted(status)) return false;
        __builtin_amdgcn_s_sleep(2);
    }
}

template <int PROTO, int DT, int CP, int U>
__global__ void __launch_bounds__(512) ring_kernel(const RingArgs a) {
    const int npos = a.hops + 1;
    const int channels = a.pipes * a.blocks_per_group;
    const int x = (int)blockIdx.x;
    int c, h;
    if (a.placement == PLACE_LOCAL) { c = x % channels; h = x / channels; }
    else                            { h = x % npos;     c = x / npos; }
    const int p = c / a.blocks_per_group;
    const int w = (c % a.blocks_per_group) * (int)(blockDim.x >> 6) + wave_in_block();
    if (w >= a.waves) return;
    const Role role = role_of(a, p, h);
    if (h == 0 && a.skip_origin) return;

    const LaneMap m;
    const uint64_t row_off = (uint64_t)p * a.row_stride;
    const uint8_t* in_row = reinterpret_cast<const uint8_t*>(a.input[role.rank]) + row_off;
    uint8_t* out_row = reinterpret_cast<uint8_t*>(a.output[role.rank]) + row_off;
    const uint32_t ring_bytes = a.nslots * a.slot_bytes;
    const Window own(reinterpret_cast<const void*>(a.staging[role.rank]), ring_bytes);
    const Window nxt(reinterpret_cast<const void*>(a.staging[role.next]), ring_bytes);
    const uint32_t chan_off = a.credit_off + ((uint32_t)p * (uint32_t)a.waves + (uint32_t)w) * kCreditStride;
    uint64_t* own_tail = reinterpret_cast<uint64_t*>(a.staging[role.rank] + chan_off);
    uint64_t* own_head = own_tail + 16;
    uint64_t* nxt_tail = reinterpret_cast<uint64_t*>(a.staging[role.next] + chan_off);
    uint64_t* nxt_head = nxt_tail + 16;

    const uint64_t flag_hi = (uint64_t)a.epoch << 32;      // credit / head words
    const uint32_t W = (uint32_t)a.waves, K = a.k_per_wave;
    uint32_t credits_seen = 0, head_seen = 0;

    for (uint32_t s = 0; s < a.steps; ++s) {
        const uint32_t slot_off = (s % a.nslots) * a.slot_bytes + (uint32_t)p * a.step_msg;
        const uint32_t g0 = s * a.step_blocks;
        const uint32_t tag = (a.epoch << 20) | (s + 1u);
        if (role.send && s >= a.nslots) {
            if (!wait_count(nxt_tail, a.epoch, s - a.nslots + 1, credits_seen, a.spin_budget,
                            a.status, false)) {
                report_timeout(a.status, p, h, w, s);
                return;
            }
        }
        if (PROTO == PROTO_SIMPLE && role.recv) {
            if (!wait_count(own_head, a.epoch, s + 1, head_seen, a.spin_budget, a.status, true)) {
                report_timeout(a.status, p, h, w, s);
                return;
            }
        }
        for (uint32_t k0 = 0; k0 < K; k0 += U) {
            uint32_t idx[U], g[U];
            bool valid[U];
            u32x4 v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                idx[u] = (k0 + (uint32_t)u) * W + (uint32_t)w;
                g[u] = g0 + idx[u];
                valid[u] = g[u] < a.nblocks;
                v[u] = u32x4{0u, 0u, 0u, 0u};
            }
            if (!valid[0]) break;
            if (role.load) {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    if (!valid[u]) continue;
                    if (PROTO == PROTO_LL128) {
                        v[u] = ll_load_raw(in_row, a.row_bytes, g[u], m);
                    } else {
                        const uint64_t off = (uint64_t)g[u] * kBlockRawSimple + m.lane * 16u;
                        v[u] = off + 16u <= a.row_bytes ? ld128_stream(in_row + off)
                                                       : load_guarded(in_row, off, 16u, a.row_bytes);
                    }
                }
            }
            if (role.recv) {
                u32x4 r[U];
                if (PROTO == PROTO_LL128) {
                    uint32_t pending = 0;
#pragma unroll
                    for (int u = 0; u < U; ++u) pending |= valid[u] ? 1u << u : 0u;
                    for (uint32_t spins = 0; pending; ++spins) {
                        compiler_fence();
#pragma unroll
                        for (int u = 0; u < U; ++u) {
                            if (!(pending & (1u << u))) continue;
                            if (ll_poll<CP>(own, slot_off + idx[u] * kBlockMsg, tag, m, r[u]))
                                pending &= ~(1u << u);
                        }
                        if (!pending) break;
                        if (spins >= a.spin_budget ||
                            ((spins & 63u) == 63u && aborted(a.status))) {
                            report_timeout(a.status, p, h, w, s);
                            return;
                        }
                        __builtin_amdgcn_s_sleep(1);
                    }
                } else {
#pragma unroll
                    for (int u = 0; u < U; ++u)
                        if (valid[u])
                            r[u] = ld128<CP>(own, slot_off + idx[u] * kBlockMsg + m.lane * 16u);
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    if (!valid[u]) continue;
                    if constexpr (DT != DT_BYTES) {
                        v[u] = role.reduce ? ll_comp<DT>(v[u], r[u]) : r[u];
                    } else {
                        v[u] = r[u];
                    }
                }
            }
            if (role.save) {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    if (!valid[u]) continue;
                    if (PROTO == PROTO_LL128) {
                        ll_save_raw(out_row, a.row_bytes, g[u], m, v[u]);
                    } else {
                        const uint64_t off = (uint64_t)g[u] * kBlockRawSimple + m.lane * 16u;
                        if (off + 16u <= a.row_bytes) st128_stream(out_row + off, v[u]);
                        else store_guarded(out_row, off, 16u, a.row_bytes, v[u]);
                    }
                }
            }
            if (role.send) {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    if (!valid[u]) continue;
                    if (PROTO == PROTO_LL128) {
                        ll_send<CP>(nxt, slot_off + idx[u] * kBlockMsg, v[u], tag, m);
                    } else {
                        st128<CP>(nxt, slot_off + idx[u] * kBlockMsg + m.lane * 16u, v[u]);
                    }
                }
            }
        }
        // post_ll128 (protocol.py:183-189): this wave-channel has taken every
        // line of step s out of its slot (the loads have returned: their
        // values were tested / used above).
        if (role.recv && lane_id() == 0) st64_agent(own_tail, flag_hi | (uint64_t)(s + 1));
        if (PROTO == PROTO_SIMPLE && role.send && lane_id() == 0)
            st64_release(nxt_head, flag_hi | (uint64_t)(s + 1));
    }
}

}  // namespace mint
