// Reduce-scatter and allgather over a hypercube of the virtual ranks.
//
// Reference: none yet - "Hypercube" is an open item of the reference's
// roadmap (README.md:52-55).  The pieces are the reference's: load / recv /
// comp / save / send of LL128 blocks (protocol.py:57-156) through circular
// staging slots with a credit word per edge (protocol.py:161-189), on the
// buffers of 7_reducescatter.py:81-98 and 6_allgather.py:141-158 (row c of
// every rank's (world, n) buffer belongs to rank c).
//
// A world of 2^d ranks; node i is rank cyc[i] (the ring order the launch
// names).  Recursive halving: in exchange k = 0 .. d-1 node i and node
// i ^ D_k, D_k = 2^(d-1-k), split the rows they are still responsible for -
// each keeps the half its own number lies in and receives the partner's
// partial sums for it.  After d exchanges node i holds row i, reduced over
// all ranks: log2(world) exchanges where the ring needs world - 1 hops.  Seen
// from one row, that is a binomial tree rooted at the row's owner: a node that
// agrees with the owner in the top m bits of its number (m = split(i, owner))
// has the children i ^ D_0 .. i ^ D_(m-1) and, unless it is the owner, the
// parent i ^ D_m.  The value a node passes on is
//     ((own + child 0) + child 1) + child 2,
// one rounding per addition, the farthest child first - the order in which
// recursive halving meets them.  Allgather is the same tree walked downwards
// (recursive doubling): a node takes a row's block from its parent, keeps it
// and sends it to its children.
//
// The `world` rows are `world` pipelines running side by side, as in the ring
// kernels; one wavefront serves one (row, node, wave-channel).  A rank
// receives world - 1 streams (reduce-scatter: one per (row, exchange) it takes
// part in as a parent; allgather: one per row that is not its own): each has
// a share of every slot and a credit word per wave-channel.
#pragma once
#include "node_step.hpp"
#include "ring.hpp"

namespace mint {

constexpr int kHyperMaxDim = 3;      // 8 ranks

__host__ __device__ __forceinline__ int hyper_dim(int world) {
    return world >= 8 ? 3 : (world >= 4 ? 2 : (world >= 2 ? 1 : 0));
}
// The exchange in which node i parts with the row of node `owner`: the first
// bit, from the top, in which their numbers differ; `dim` for the owner itself.
__host__ __device__ __forceinline__ int hyper_split(int i, int owner, int dim) {
    for (int k = 0; k < dim; ++k)
        if ((i ^ owner) & (1 << (dim - 1 - k))) return k;
    return dim;
}
// Share of node `to`'s slots that carries row `owner`'s blocks
// sent in exchange k of a reduce-scatter: the streams of exchange k are the
// D_k rows the node still holds then, numbered behind those of the later
// exchanges (D - 1 + the row's number relative to the node, below D).
__host__ __device__ __forceinline__ uint32_t hyper_share_up(int to, int owner, int k, int dim) {
    const int D = 1 << (dim - 1 - k);
    return (uint32_t)(D - 1 + ((owner ^ to) & (D - 1)));
}
// ... and of an allgather: one stream per row that is not the node's own.
__host__ __device__ __forceinline__ uint32_t hyper_share_down(int to, int owner) {
    return (uint32_t)((owner ^ to) - 1);
}

template <int DT, int CPI>
__device__ __forceinline__ void hyper_walk(const RingArgs& a, const int p, const int h,
                                           const int w) {
    constexpr int LDCP = Policy<CPI>::LD, STCP = Policy<CPI>::ST;
    const LaneMap m;
    const bool up = a.op == OP_HYPER_REDUCESCATTER;
    const int dim = hyper_dim(a.world);
    const int owner = a.start[p];                    // node that row p belongs to
    const int split = hyper_split(h, owner, dim);    // children: exchanges 0 .. split - 1
    const int rank = a.cyc[h];
    // data flows up the row's tree in a reduce-scatter, down in an allgather
    const int nin = up ? split : (h == owner ? 0 : 1);
    const int nout = up ? (h == owner ? 0 : 1) : split;
    const bool load = up || h == owner;
    const bool save = up ? h == owner : h != owner;

    uint64_t row_bytes;
    uint32_t nblocks, nfull;
    row_extent(a, p, kBlockRawLL, row_bytes, nblocks, nfull);
    const uint8_t* in_row = reinterpret_cast<const uint8_t*>(a.input[rank]) + (uint64_t)p * a.row_stride;
    uint8_t* out_row = reinterpret_cast<uint8_t*>(a.output[rank]) + (uint64_t)p * a.row_stride;
    const uint32_t ring_bytes = a.nslots * a.slot_bytes;
    const uint32_t W = (uint32_t)a.waves, K = a.k_per_wave;

    // where this node sends (up to three places), and which shares it receives in
    int to[kHyperMaxDim];
    uint32_t to_share[kHyperMaxDim], in_share[kHyperMaxDim];
#pragma unroll
    for (int j = 0; j < kHyperMaxDim; ++j) {
        const int D = 1 << (dim - 1 - (j < dim ? j : dim - 1));
        if (up) {
            const int parent = h == owner ? h : h ^ (1 << (dim - 1 - split));
            to[j] = a.cyc[parent];
            to_share[j] = h == owner ? 0u : hyper_share_up(parent, owner, split, dim);
            in_share[j] = j < split ? hyper_share_up(h, owner, j, dim) : 0u;
        } else {
            const int child = j < split ? h ^ D : h;
            to[j] = a.cyc[child];
            to_share[j] = j < split ? hyper_share_down(child, owner) : 0u;
            in_share[j] = h == owner ? 0u : hyper_share_down(h, owner);
        }
    }
    const Window own(reinterpret_cast<const void*>(a.staging[rank]), ring_bytes);
    const Window out0(reinterpret_cast<const void*>(a.staging[to[0]]), ring_bytes);
    const Window out1(reinterpret_cast<const void*>(a.staging[to[1]]), ring_bytes);
    const Window out2(reinterpret_cast<const void*>(a.staging[to[2]]), ring_bytes);
    auto credit_word = [&](int of_rank, uint32_t share) {
        return reinterpret_cast<uint64_t*>(a.staging[of_rank] + a.credit_off +
                                           (share * W + (uint32_t)w) * kCreditStride);
    };
    uint64_t* const in_tail[kHyperMaxDim] = {credit_word(rank, in_share[0]), credit_word(rank, in_share[1]),
                                             credit_word(rank, in_share[2])};
    const uint64_t* const out_tail[kHyperMaxDim] = {credit_word(to[0], to_share[0]),
                                                    credit_word(to[1], to_share[1]),
                                                    credit_word(to[2], to_share[2])};

    const uint32_t epoch = launch_epoch(a);
    const uint64_t flag_hi = (uint64_t)epoch << 32;
    uint32_t credits_seen[kHyperMaxDim] = {0u, 0u, 0u};

    // The whole steps of the tuned launches (one block per wave-channel and
    // step, XCD-local staging) run in the loop of node_step.hpp, chosen by the
    // node's shape; what is left, and every other launch, takes the loop below.
    uint32_t s_begin = 0;
    if constexpr (CPI == 2) {
        uint32_t whole = nfull > (uint32_t)w ? (nfull - 1u - (uint32_t)w) / a.step_blocks + 1u : 0u;
        if (whole > a.steps) whole = a.steps;
        if (K == 1u && whole && up == (DT != DT_BYTES)) {
            NodeEdges e;
#pragma unroll
            for (int j = 0; j < kHyperMaxDim; ++j) {
                e.in_off[j] = in_share[j] * a.step_msg;
                e.out_off[j] = to_share[j] * a.step_msg;
                e.in_tail[j] = in_tail[j];
                e.out_tail[j] = out_tail[j];
            }
#define MINT_NODE(UP_, NIN_, NOUT_)                                                              \
    if (nin == NIN_ && nout == NOUT_) {                                                          \
        node_whole_steps<DT, CPI, UP_, NIN_, NOUT_>(a, p, h, w, whole, own, out0, out1, out2, e, \
                                                    in_row, out_row, row_bytes, nfull,           \
                                                    credits_seen);                               \
        s_begin = whole;                                                                         \
    }
            if constexpr (DT != DT_BYTES) {
                MINT_NODE(true, 0, 1) else MINT_NODE(true, 1, 1) else MINT_NODE(true, 2, 1)
                else MINT_NODE(true, 1, 0) else MINT_NODE(true, 2, 0) else MINT_NODE(true, 3, 0)
            } else {
                MINT_NODE(false, 0, 1) else MINT_NODE(false, 0, 2) else MINT_NODE(false, 0, 3)
                else MINT_NODE(false, 1, 0) else MINT_NODE(false, 1, 1) else MINT_NODE(false, 1, 2)
            }
#undef MINT_NODE
        }
    }

    // Own rows one block ahead (whole blocks only; the ragged last block of a
    // row is loaded where it is used): the load from HBM is in flight while
    // the block before it is polled for, added and sent.
    const uint32_t last_k = K - 1u;
    u32x4 ahead = {0u, 0u, 0u, 0u};
    if (load && s_begin == 0u && (uint32_t)w < nfull)
        ahead = ll_fetch_raw(in_row, row_bytes, (uint32_t)w, true, m);

    uint32_t slot = s_begin % a.nslots;
    for (uint32_t s = s_begin; s < a.steps; ++s) {
        const uint32_t tag = (epoch << 20) | (s + 1u);
        // wait_ll128 (protocol.py:161-180): the receivers have emptied the slot
        // this step goes into
        const uint32_t need = s >= a.nslots ? s - a.nslots + 1 : 0;
#pragma unroll
        for (int j = 0; j < kHyperMaxDim; ++j)
            if (j < nout && !wait_count(out_tail[j], epoch, need, credits_seen[j], a.spin_budget,
                                        a.status)) {
                report_timeout(a.status, p, h, w, s);
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
            u32x4 r[kHyperMaxDim];
            uint32_t pending = 0;
            compiler_fence();
#pragma unroll
            for (int j = 0; j < kHyperMaxDim; ++j)
                if (j < nin) r[j] = ld128<LDCP>(own, at + in_share[j] * a.step_msg + m.lane * 16u);
            // the wave-channel's next block: k + 1 of this step, or block 0 of the next
            {
                const uint32_t gn = k < last_k ? g + W : (s + 1u) * a.step_blocks + (uint32_t)w;
                if (load && gn < nfull) ahead = ll_fetch_raw(in_row, row_bytes, gn, true, m);
            }
#pragma unroll
            for (int j = 0; j < kHyperMaxDim; ++j)
                if (j < nin && !wave_all(!m.flag_lane || r[j].w == tag)) pending |= 1u << j;
            for (uint32_t spins = 0; pending; ++spins) {
                if (spins >= a.spin_budget || ((spins & 63u) == 63u && aborted(a.status))) {
                    report_timeout(a.status, p, h, w, s);
                    return;
                }
                __builtin_amdgcn_s_sleep(1);
                compiler_fence();
#pragma unroll
                for (int j = 0; j < kHyperMaxDim; ++j)
                    if ((pending & (1u << j)) &&
                        ll_poll<LDCP>(own, at + in_share[j] * a.step_msg, tag, m, r[j]))
                        pending &= ~(1u << j);
            }
            // recv + comp (protocol.py:102-156): the farthest child first
#pragma unroll
            for (int j = 0; j < kHyperMaxDim; ++j) {
                if (j >= nin) continue;
                if constexpr (DT != DT_BYTES) {
                    x = up ? ll_comp<DT>(x, r[j]) : r[j];
                } else {
                    x = r[j];
                }
            }
            if (save) ll_save_raw(out_row, row_bytes, g, m, x);
            if (nout > 0) ll_send<STCP>(out0, at + to_share[0] * a.step_msg, x, tag, m);
            if (nout > 1) ll_send<STCP>(out1, at + to_share[1] * a.step_msg, x, tag, m);
            if (nout > 2) ll_send<STCP>(out2, at + to_share[2] * a.step_msg, x, tag, m);
        }
        // post_ll128 (protocol.py:183-189): every block of step s has been
        // taken out of this node's slots (the polls tested what they loaded)
        if (lane_id() == 0) {
#pragma unroll
            for (int j = 0; j < kHyperMaxDim; ++j) {
                if (j >= nin) continue;
                if (STCP == CP_NONE) st64_local(in_tail[j], flag_hi | (uint64_t)(s + 1));
                else st64_agent(in_tail[j], flag_hi | (uint64_t)(s + 1));
            }
        }
        slot = slot + 1 == a.nslots ? 0 : slot + 1;
    }
}

// Seats are dealt as for the ring kernels (position = node), so with the local
// placement a wave-channel's whole tree shares one XCD.
template <int DT, int CPI>
__global__ void __launch_bounds__(512) hyper_kernel(const RingArgs a) {
    __shared__ int entry[1];
    const int wpb = (int)(blockDim.x >> 6);
    const int wib = (int)__builtin_amdgcn_readfirstlane((uint32_t)wave_in_block());
    const Seat st = take_seat(a, wpb, wib, wib, (MINT_LDS int*)entry);
    if (!st.ok) return;
    hyper_walk<DT, CPI>(a, st.p, st.h, st.w);
}

}  // namespace mint
