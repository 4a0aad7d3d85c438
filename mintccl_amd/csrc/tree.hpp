// Broadcast and reduce over a binary tree of the virtual ranks.
//
// Reference: none yet - "Tree / Binary Tree" is an open item of the
// reference's roadmap (README.md:52-55).  The pieces are the reference's:
// load / recv / comp / save / send of LL128 blocks in the order of
// 4_broadcast.py:55-70 and 5_reduce.py:70-89, through circular staging slots
// with a credit word per edge (protocol.py:161-189).
//
// The tree is laid over the ring order the launch names, turned so that the
// root comes first: node h (0 = root) is rank cyc[(start + h) % world], its
// parent is node (h - 1) / 2, its children are nodes 2h + 1 and 2h + 2 where
// they exist.  Eight ranks are three hops deep where the ring is seven.
//
//   broadcast  a node takes a block from its parent's send (the root: from
//              its own buffer), keeps a copy (all but the root) and sends it
//              to both children
//   reduce     a node adds to its own block the block of its first child,
//              then that of its second child, one rounding each, and sends
//              the sum to its parent (the root: stores it)
//
// so the value a node passes up is  (own + first subtree) + second subtree.
//
// One wavefront serves one (node, wave-channel) and does everything that node
// does with the wave-channel's blocks; wave-channel w of a node talks only to
// wave-channel w of its parent and children, as on the ring.  A node that
// receives from two children has two shares in each of its slots, one per
// child, and a credit word for each.
#pragma once
#include "node_step.hpp"
#include "ring.hpp"

namespace mint {

constexpr int kTreeArity = 2;

__host__ __device__ __forceinline__ int tree_rank(const RingArgs& a, int h) {
    return a.cyc[(a.start[0] + h) % a.world];
}
__host__ __device__ __forceinline__ int tree_children(int h, int world) {
    const int c = world - (kTreeArity * h + 1);
    return c < 0 ? 0 : (c > kTreeArity ? kTreeArity : c);
}

template <int DT, int CPI>
__device__ __forceinline__ void tree_walk(const RingArgs& a, const int h, const int w) {
    constexpr int LDCP = Policy<CPI>::LD, STCP = Policy<CPI>::ST;
    const LaneMap m;
    const bool reduce = a.op == OP_TREE_REDUCE;
    const int rank = tree_rank(a, h);
    const int nchild = tree_children(h, a.world);
    // data flows down the tree in a broadcast, up in a reduce
    const int nin = reduce ? nchild : (h ? 1 : 0);
    const int nout = reduce ? (h ? 1 : 0) : nchild;
    const bool load = reduce || h == 0;
    const bool save = reduce ? h == 0 : h != 0;

    const uint64_t row_bytes = a.row_bytes;
    const uint32_t nblocks = a.nblocks;
    const uint8_t* in_row = reinterpret_cast<const uint8_t*>(a.input[rank]);
    uint8_t* out_row = reinterpret_cast<uint8_t*>(a.output[rank]);
    const uint32_t ring_bytes = a.nslots * a.slot_bytes;
    const uint32_t W = (uint32_t)a.waves, K = a.k_per_wave;

    // where this node sends: rank, and which share of that rank's slots
    int to[kTreeArity];
    uint32_t to_share[kTreeArity];
#pragma unroll
    for (int j = 0; j < kTreeArity; ++j) {
        if (reduce) {
            to[j] = h ? tree_rank(a, (h - 1) / kTreeArity) : rank;
            to_share[j] = h ? (uint32_t)((h - 1) % kTreeArity) : 0u;
        } else {
            to[j] = j < nchild ? tree_rank(a, kTreeArity * h + 1 + j) : rank;
            to_share[j] = 0u;
        }
    }
    const Window own(reinterpret_cast<const void*>(a.staging[rank]), ring_bytes);
    const Window out0(reinterpret_cast<const void*>(a.staging[to[0]]), ring_bytes);
    const Window out1(reinterpret_cast<const void*>(a.staging[to[1]]), ring_bytes);
    auto credit_word = [&](int of_rank, uint32_t share) {
        return reinterpret_cast<uint64_t*>(a.staging[of_rank] + a.credit_off +
                                           (share * W + (uint32_t)w) * kCreditStride);
    };
    uint64_t* const in_tail[kTreeArity] = {credit_word(rank, 0u), credit_word(rank, 1u)};
    const uint64_t* const out_tail[kTreeArity] = {credit_word(to[0], to_share[0]),
                                                  credit_word(to[1], to_share[1])};

    const uint32_t epoch = launch_epoch(a);
    const uint64_t flag_hi = (uint64_t)epoch << 32;

    uint32_t credits_seen[kTreeArity] = {0u, 0u};

    // Own rows one block ahead (whole blocks only; the ragged last block of a
    // row is loaded where it is used): the load from HBM is in flight while
    // the block before it is polled for, added and sent.
    const uint32_t nfull = (uint32_t)(row_bytes / kBlockRawLL);
    const uint32_t last_k = K - 1u;
    u32x4 ahead = {0u, 0u, 0u, 0u};
    if (load && (uint32_t)w < nfull) ahead = ll_fetch_raw(in_row, row_bytes, (uint32_t)w, true, m);

    uint32_t slot = 0, s = 0;
    if (!reduce && h == 0 && STCP == CP_NONE && K == 1u && nout > 0) {
        // The root of a broadcast, one block per step, XCD-local staging, on
        // compute units set apart for it (origin_cus): rows fetched kAhead
        // steps ahead, the children's credit words read through the scalar
        // unit so that looking at them does not wait for the fetches (a load
        // from HBM takes 2.5 us under the tree's stores).  Whole blocks only;
        // the ragged end of the buffer takes the loop below.
        constexpr uint32_t kAhead = 4;
        const uint32_t whole = nfull > (uint32_t)w ? (nfull - 1u - (uint32_t)w) / a.step_blocks + 1u : 0u;
        const uint32_t deep = whole < a.steps ? whole : a.steps;
        if (deep) {
            u32x4 vv[kAhead];
            auto fetch = [&](uint32_t of_step) __attribute__((always_inline)) {
                uint32_t g = of_step * a.step_blocks + (uint32_t)w;
                g = g < nfull ? g : nfull - 1u;              // beyond the whole blocks: any valid address
                return ll_fetch_raw(in_row, row_bytes, g, true, m);
            };
            // (the prologue issues the queue a later step finds: stores stand in
            // for a step's two sends, to an unused part of a credit line)
            uint64_t* const pad = const_cast<uint64_t*>(out_tail[0]) + 8;
            vv[0] = fetch(0u);
#pragma unroll
            for (uint32_t d = 1; d < kAhead; ++d) {
                compiler_fence();
                st64_local(pad, 0ull);
                st64_local(pad, 0ull);
                compiler_fence();
                vv[d] = fetch(d);
            }
            auto step = [&](auto phase) __attribute__((always_inline)) {
                constexpr int B = decltype(phase)::value;
                const uint32_t tag = (epoch << 20) | (s + 1u);
                const uint32_t need = s >= a.nslots ? s - a.nslots + 1 : 0;
#pragma unroll
                for (int j = 0; j < kTreeArity; ++j) {
                    if (j >= nout) continue;
                    for (uint32_t spins = 0; credits_seen[j] < need; ++spins) {
                        const uint64_t cw = ld64_scalar(out_tail[j]);
                        if ((uint32_t)(cw >> 32) == epoch && (uint32_t)cw >= need) {
                            credits_seen[j] = (uint32_t)cw;
                            break;
                        }
                        if (spins >= a.spin_budget ||
                            ((spins & 63u) == 63u &&
                             __builtin_amdgcn_readfirstlane(ld32_agent_apart(a.status + 3)) != 0u)) {
                            report_timeout(a.status, 0, h, w, s);
                            __builtin_amdgcn_endpgm();
                        }
                        __builtin_amdgcn_s_sleep(1);
                    }
                }
                const uint32_t at = slot * a.slot_bytes + (uint32_t)w * kBlockMsg;
                const u32x4 x = ll_arrange(vv[B], true, m);
                // (a root with one child sends the block twice to the same place)
                ll_send<STCP>(out0, at, x, tag, m);
                ll_send<STCP>(nout > 1 ? out1 : out0, at, x, tag, m);
                compiler_fence();
                vv[B] = fetch(s + kAhead);
                slot = slot + 1 == a.nslots ? 0 : slot + 1;
                ++s;
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
            // the loop below fetches its own rows one block ahead
            if (s < a.steps) {
                const uint32_t g = s * a.step_blocks + (uint32_t)w;
                if (g < nfull) ahead = ll_fetch_raw(in_row, row_bytes, g, true, m);
            }
        }
    } else if constexpr (CPI == 2) {
        // Every other node of a tuned launch (one block per wave-channel and
        // step, XCD-local staging): its whole steps run in the loop of
        // node_step.hpp, chosen by the node's shape.
        uint32_t whole = nfull > (uint32_t)w ? (nfull - 1u - (uint32_t)w) / a.step_blocks + 1u : 0u;
        if (whole > a.steps) whole = a.steps;
        if (K == 1u && whole && reduce == (DT != DT_BYTES)) {
            NodeEdges e;
            uint32_t seen[kNodeMaxEdges] = {credits_seen[0], credits_seen[1], 0u};
#pragma unroll
            for (int j = 0; j < kNodeMaxEdges; ++j) {
                const int i = j < kTreeArity ? j : 0;
                e.in_off[j] = (uint32_t)i * a.step_msg;
                e.out_off[j] = to_share[i] * a.step_msg;
                e.in_tail[j] = in_tail[i];
                e.out_tail[j] = out_tail[i];
            }
            bool done = false;
#define MINT_NODE(UP_, NIN_, NOUT_)                                                               \
    if (nin == NIN_ && nout == NOUT_) {                                                           \
        node_whole_steps<DT, CPI, UP_, NIN_, NOUT_>(a, 0, h, w, whole, own, out0, out1, out1, e,  \
                                                    in_row, out_row, row_bytes, nfull, seen);     \
        done = true;                                                                              \
    }
            if constexpr (DT != DT_BYTES) {
                MINT_NODE(true, 0, 1) else MINT_NODE(true, 1, 1) else MINT_NODE(true, 2, 1)
                else MINT_NODE(true, 1, 0) else MINT_NODE(true, 2, 0)
            } else {
                // (the root has the loop above)
                MINT_NODE(false, 1, 0) else MINT_NODE(false, 1, 1) else MINT_NODE(false, 1, 2)
            }
#undef MINT_NODE
            if (done) {
                credits_seen[0] = seen[0];
                credits_seen[1] = seen[1];
                s = whole;
                slot = whole % a.nslots;
            }
        }
    }
    for (; s < a.steps; ++s) {
        const uint32_t tag = (epoch << 20) | (s + 1u);
        // wait_ll128 (protocol.py:161-180): the receiver has emptied the slot
        // this step goes into
        const uint32_t need = s >= a.nslots ? s - a.nslots + 1 : 0;
#pragma unroll
        for (int j = 0; j < kTreeArity; ++j)
            if (j < nout && !wait_count(out_tail[j], epoch, need, credits_seen[j], a.spin_budget,
                                        a.status)) {
                report_timeout(a.status, 0, h, w, s);
                return;
            }
        for (uint32_t k = 0; k < K; ++k) {
            const uint32_t idx = k * W + (uint32_t)w;
            const uint32_t g = s * a.step_blocks + idx;
            if (g >= nblocks) break;
            const uint32_t at = slot * a.slot_bytes + idx * kBlockMsg;
            u32x4 x = {0u, 0u, 0u, 0u};
            if (load) x = g < nfull ? ll_arrange(ahead, true, m) : ll_load_raw(in_row, row_bytes, g, m);
            // first poll of every incoming block at once, then the repeats
            u32x4 r[kTreeArity];
            uint32_t pending = 0;
            compiler_fence();
#pragma unroll
            for (int j = 0; j < kTreeArity; ++j)
                if (j < nin) r[j] = ld128<LDCP>(own, at + (uint32_t)j * a.step_msg + m.lane * 16u);
            // the wave-channel's next block: k + 1 of this step, or block 0 of the next
            {
                const uint32_t gn = k < last_k ? g + W : (s + 1u) * a.step_blocks + (uint32_t)w;
                if (load && gn < nfull) ahead = ll_fetch_raw(in_row, row_bytes, gn, true, m);
            }
#pragma unroll
            for (int j = 0; j < kTreeArity; ++j)
                if (j < nin && !wave_all(!m.flag_lane || r[j].w == tag)) pending |= 1u << j;
            for (uint32_t spins = 0; pending; ++spins) {
                if (spins >= a.spin_budget || ((spins & 63u) == 63u && aborted(a.status))) {
                    report_timeout(a.status, 0, h, w, s);
                    return;
                }
                __builtin_amdgcn_s_sleep(1);
                compiler_fence();
#pragma unroll
                for (int j = 0; j < kTreeArity; ++j)
                    if ((pending & (1u << j)) &&
                        ll_poll<LDCP>(own, at + (uint32_t)j * a.step_msg, tag, m, r[j]))
                        pending &= ~(1u << j);
            }
#pragma unroll
            for (int j = 0; j < kTreeArity; ++j) {
                if (j >= nin) continue;
                if constexpr (DT != DT_BYTES) {
                    x = reduce ? ll_comp<DT>(x, r[j]) : r[j];
                } else {
                    x = r[j];
                }
            }
            if (save) ll_save_raw(out_row, row_bytes, g, m, x);
            if (nout > 0) ll_send<STCP>(out0, at + to_share[0] * a.step_msg, x, tag, m);
            if (nout > 1) ll_send<STCP>(out1, at + to_share[1] * a.step_msg, x, tag, m);
        }
        // post_ll128 (protocol.py:183-189): every block of step s has been
        // taken out of this node's slot (the polls tested what they loaded)
        if (lane_id() == 0) {
#pragma unroll
            for (int j = 0; j < kTreeArity; ++j) {
                if (j >= nin) continue;
                if (STCP == CP_NONE) st64_local(in_tail[j], flag_hi | (uint64_t)(s + 1));
                else st64_agent(in_tail[j], flag_hi | (uint64_t)(s + 1));
            }
        }
        slot = slot + 1 == a.nslots ? 0 : slot + 1;
    }
}

// Seats are dealt as for the ring kernels (position = node of the tree), so
// with the local placement a wave-channel's whole tree shares one XCD.
template <int DT, int CPI>
__global__ void __launch_bounds__(512) tree_kernel(const RingArgs a) {
    __shared__ int entry[1];
    const int wpb = (int)(blockDim.x >> 6);
    const int wib = (int)__builtin_amdgcn_readfirstlane((uint32_t)wave_in_block());
    const Seat st = take_seat(a, wpb, wib, wib, (MINT_LDS int*)entry);
    if (!st.ok) return;
    tree_walk<DT, CPI>(a, st.h, st.w);
}

}  // namespace mint
