// libmintccl.so - C ABI over the HIP kernels (see include/mintccl.h).
#include "../../include/mintccl.h"

#include <hip/hip_runtime.h>

#include <atomic>

#include "kernels.hpp"
#include "ring_launch.hpp"
#include "hypercube.hpp"
#include "temporal.hpp"
#include "tree.hpp"

using namespace mint;

// Staging for mint_ring_launch_static: slots, credit words and the launch epoch
// of all ranks, in device memory that exists from the moment the library is
// loaded.  Every GPU the library runs on holds its own copy at its own
// address.  In host code the name `scratch` only identifies the symbol; the
// device address comes from hipGetSymbolAddress, once per device.
//   [0, 4096)                              header: word 0 = launch epoch, word 1 = protocol
//                                          of the launch before (+ 1; 0 = none yet)
//   4096 + r * MINT_STATIC_RANK_BYTES      rank r: [slots ... | credit words (last 256 KiB)]
static __device__ __align__(256) unsigned char scratch[MINT_STATIC_SCRATCH_BYTES];

namespace {

constexpr int kVersion = 102;   // 0.1.2: mint_build_flags, mint_static_init, mint_step_mix_deep,
                                // mint_ring_seat, the hypercube ops; mint_epoch_advance takes the
                                // protocol; staging grew by the seat counters
// What this library was compiled with (mint_build_flags).
constexpr int kBuildFlags = 0
#ifdef MINT_RING_STATS
                            | MINT_BUILD_RING_STATS
#endif
#ifdef MINT_ROW_NOLOAD
                            | MINT_BUILD_ROW_NOLOAD
#endif
    ;
constexpr uint32_t kDefaultSpinBudget = 4000000u;
constexpr uint32_t kMaxEpoch = 4095u;          // 12 bits of every sector tag
constexpr uint32_t kMaxSteps = (1u << 20) - 1; // 20 bits of every sector tag
constexpr uint32_t kFetchDepth = 4;            // own rows through LDS: groups of LDS per wave-channel

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }
inline bool aligned16(uint64_t p) { return (p & 15u) == 0; }
inline bool aligned16(const void* p) { return aligned16(reinterpret_cast<uint64_t>(p)); }

bool reducing(int op) {
    return op == MINT_OP_REDUCE || op == MINT_OP_REDUCESCATTER || op == MINT_OP_ALLREDUCE ||
           op == MINT_OP_TREE_REDUCE || op == MINT_OP_HYPERCUBE_REDUCESCATTER;
}
bool over_hypercube(int op) {
    return op == MINT_OP_HYPERCUBE_REDUCESCATTER || op == MINT_OP_HYPERCUBE_ALLGATHER;
}
bool over_tree(int op) { return op == MINT_OP_TREE_BROADCAST || op == MINT_OP_TREE_REDUCE; }
static_assert(MINT_OP_TREE_BROADCAST == OP_TREE_BROADCAST && MINT_OP_TREE_REDUCE == OP_TREE_REDUCE &&
                  MINT_OP_ALLGATHER_TEMPORAL == OP_ALLGATHER_TEMPORAL &&
                  MINT_OP_HYPERCUBE_REDUCESCATTER == OP_HYPER_REDUCESCATTER &&
                  MINT_OP_HYPERCUBE_ALLGATHER == OP_HYPER_ALLGATHER,
              "op codes");

// Everything the launch derives from the descriptor.  `for_launch`: also
// check what only matters once the kernels run (the size of the staging the
// caller allocated); the host-side queries do without.
int make_plan(const mint_ring_op* op, Plan* plan, bool for_launch = false,
              const mint_ring_debug* dbg = nullptr) {
    if (!op || !plan) return MINT_ERR_ARG;
    if (op->op < MINT_OP_SENDRECV || op->op > MINT_OP_HYPERCUBE_ALLGATHER) return MINT_ERR_ARG;
    if (op->protocol != MINT_PROTO_LL128 && op->protocol != MINT_PROTO_SIMPLE) return MINT_ERR_ARG;
    if (op->world < 1 || op->world > MINT_MAX_RANKS) return MINT_ERR_ARG;
    // the tree kernels and the temporal allgather speak LL128 only
    const bool temporal = op->op == MINT_OP_ALLGATHER_TEMPORAL;
    const bool hyper = over_hypercube(op->op);
    if ((over_tree(op->op) || temporal || hyper) && op->protocol != MINT_PROTO_LL128)
        return MINT_ERR_ARG;
    // a hypercube has 2^d corners
    if (hyper && (op->world & (op->world - 1))) return MINT_ERR_ARG;
    if (op->dtype < MINT_F16 || op->dtype > MINT_BYTES) return MINT_ERR_ARG;
    if (reducing(op->op) && op->dtype == MINT_BYTES) return MINT_ERR_ARG;
    if (op->cache_policy < 0 || op->cache_policy > 2) return MINT_ERR_ARG;
    // XCD-local staging only makes sense when every hop of a channel shares an XCD
    if (op->cache_policy == 2 && op->placement != MINT_PLACE_LOCAL) return MINT_ERR_ARG;
    if (op->placement != MINT_PLACE_SPREAD && op->placement != MINT_PLACE_LOCAL) return MINT_ERR_ARG;
    if (op->row_fetch != MINT_FETCH_INLINE && op->row_fetch != MINT_FETCH_LDS) return MINT_ERR_ARG;
    if (!op->status) return MINT_ERR_ARG;
    if (op->epoch_ptr) {
        if (op->epoch_ptr % 4) return MINT_ERR_ALIGN;        // the epoch lives in device memory
    } else if (op->flag_epoch == 0 || op->flag_epoch > kMaxEpoch) {
        return MINT_ERR_ARG;
    }
    if (op->threads_per_block == 0 || op->threads_per_block % 64 || op->threads_per_block > 512)
        return MINT_ERR_ARG;
    if (op->nslots == 0 || op->slot_bytes == 0) return MINT_ERR_GEOMETRY;
    if ((uint64_t)op->nslots * op->slot_bytes >= (1ull << 31)) return MINT_ERR_TOO_LARGE;

    RingArgs& a = plan->args;
    a = RingArgs{};
    a.op = op->op;
    a.world = op->world;
    const bool allreduce = op->op == MINT_OP_ALLREDUCE;
    const bool alltoall = op->op == MINT_OP_ALLTOALL;
    const bool rowwise = op->op == MINT_OP_ALLGATHER || op->op == MINT_OP_REDUCESCATTER ||
                         allreduce || alltoall || temporal || hyper;
    // (the temporal allgather moves its `world` rows one after the other
    // through one pipeline)
    a.pipes = alltoall ? op->world * op->world : (rowwise && !temporal ? op->world : 1);
    a.phases = allreduce ? 2 : 1;
    // a rank receives from every pipeline that passes through it: one share of
    // its slots per pipeline and phase; in an alltoall, one per source rank
    a.shares = alltoall ? op->world : a.pipes * a.phases;
    // a node of a reducing tree receives from two children: a share of its slots each
    if (op->op == MINT_OP_TREE_REDUCE) a.shares = kTreeArity;
    // a corner of a hypercube receives world - 1 streams (hypercube.hpp)
    if (hyper) a.shares = op->world > 1 ? op->world - 1 : 1;

    // ring / route
    bool seen[MINT_MAX_RANKS] = {};
    if (op->op == MINT_OP_SENDRECV) {
        if (op->route_len < 1 || op->route_len > op->world) return MINT_ERR_ARG;
        a.cyc_len = op->route_len;
    } else {
        a.cyc_len = op->world;
        // (an alltoall sends every row straight to its destination: the ring
        // is not walked, but it still has to be one)
        if (op->ring[op->world] != op->ring[0]) return MINT_ERR_ARG;
    }
    for (int i = 0; i < a.cyc_len; ++i) {
        int r = op->ring[i];
        if (r < 0 || r >= op->world || seen[r]) return MINT_ERR_ARG;
        seen[r] = true;
        a.cyc[i] = (uint8_t)r;
    }
    auto index_of = [&](int rank) {
        for (int i = 0; i < a.cyc_len; ++i) if (a.cyc[i] == rank) return i;
        return -1;
    };
    switch (op->op) {
        case MINT_OP_SENDRECV:  a.hops = a.cyc_len - 1; a.start[0] = 0; break;
        case MINT_OP_BROADCAST:
        case MINT_OP_REDUCE:
        case MINT_OP_TREE_BROADCAST:
        case MINT_OP_TREE_REDUCE: {
            if (op->root < 0 || op->root >= op->world) return MINT_ERR_ARG;
            // (a tree has one position per node)
            a.hops = op->op == MINT_OP_REDUCE ? op->world : op->world - 1;
            a.start[0] = (uint8_t)index_of(op->root);
            break;
        }
        case MINT_OP_ALLTOALL: a.hops = 1; break;
        default:
            a.hops = op->op == MINT_OP_ALLGATHER || temporal || hyper ? op->world - 1
                     : allreduce                             ? 2 * op->world - 2
                                                             : op->world;
            for (int p = 0; p < op->world; ++p) a.start[p] = (uint8_t)index_of(p);
    }

    const int dt_size = op->dtype == MINT_F32 ? 4 : (op->dtype == MINT_BYTES ? 1 : 2);
    if (op->count_bytes % dt_size) return MINT_ERR_ARG;
    if (allreduce) {
        if (op->total_bytes) return MINT_ERR_ARG;
        // one buffer of count_bytes per rank, cut into `world` rows of whole
        // 16-byte vectors; the last rows may be short or empty
        const uint64_t per = (op->count_bytes + op->world - 1) / op->world;
        a.row_bytes = (per + 15) / 16 * 16;
        a.row_stride = a.row_bytes;
        a.total_bytes = op->count_bytes;
    } else {
        a.row_bytes = op->count_bytes;
        a.row_stride = rowwise ? op->row_stride : 0;
        if (rowwise && op->row_stride < op->count_bytes) return MINT_ERR_ARG;   // rows overlap
        if (op->total_bytes) {
            // rows cut from one buffer: the last ones may be short or empty
            if (!rowwise || alltoall || op->total_bytes % dt_size ||
                op->total_bytes > (uint64_t)op->world * op->row_stride)
                return MINT_ERR_ARG;
            a.total_bytes = op->total_bytes;
        }
    }
    plan->empty = op->count_bytes == 0 || op->world == 1 ||
                  (op->op == MINT_OP_SENDRECV && a.cyc_len == 1);

    // which ranks need which buffers
    for (int h = 0; h < op->world && over_tree(op->op) && !plan->empty; ++h) {
        const int rank = tree_rank(a, h);
        const bool up = op->op == MINT_OP_TREE_REDUCE;
        const bool receives = up ? tree_children(h, op->world) > 0 : h != 0;
        if ((up || h == 0) && !op->input[rank]) return MINT_ERR_ARG;
        if ((up ? h == 0 : h != 0) && !op->output[rank]) return MINT_ERR_ARG;
        if (receives && (!op->staging[rank] || !aligned16(op->staging[rank])))
            return op->staging[rank] ? MINT_ERR_ALIGN : MINT_ERR_ARG;
    }
    for (int r = 0; r < op->world && (temporal || hyper) && !plan->empty; ++r) {
        // every rank is origin once and receiver world - 1 times
        if (!op->input[r] || !op->output[r]) return MINT_ERR_ARG;
        if (!op->staging[r] || !aligned16(op->staging[r]))
            return op->staging[r] ? MINT_ERR_ALIGN : MINT_ERR_ARG;
    }
    for (int p = 0; p < a.pipes && !plan->empty && !over_tree(op->op) && !temporal && !hyper; ++p) {
        for (int h = 0; h <= a.hops; ++h) {
            const int rank = alltoall ? (h == 0 ? p / op->world : p % op->world)
                                      : a.cyc[(a.start[p] + h) % a.cyc_len];
            const bool origin = h == 0, sink = h == a.hops;
            const bool load = allreduce ? h < op->world : origin || (reducing(op->op) && !sink);
            const bool save = allreduce ? h >= op->world - 1
                                        : sink || ((op->op == MINT_OP_BROADCAST ||
                                                    op->op == MINT_OP_ALLGATHER) && !origin);
            // caller buffers and rows may start at any byte; staging is ours
            if (load && !op->input[rank]) return MINT_ERR_ARG;
            if (save && !op->output[rank]) return MINT_ERR_ARG;
            if (!origin && (!op->staging[rank] || !aligned16(op->staging[rank])))
                return op->staging[rank] ? MINT_ERR_ALIGN : MINT_ERR_ARG;
        }
    }
    if (alltoall && !plan->empty) {
        // every row is read while others are written: no output may overlap an input
        const uint64_t extent = (uint64_t)(op->world - 1) * op->row_stride + op->count_bytes;
        for (int i = 0; i < op->world; ++i)
            for (int o = 0; o < op->world; ++o)
                if (op->input[i] < op->output[o] + extent && op->output[o] < op->input[i] + extent)
                    return MINT_ERR_ARG;
    }
    for (int r = 0; r < op->world; ++r) {
        a.input[r] = op->input[r];
        a.output[r] = op->output[r];
        a.staging[r] = op->staging[r];
    }

    // geometry
    a.slot_bytes = op->slot_bytes;
    a.nslots = op->nslots;
    // a slot is shared evenly by the pipelines, in whole 1 KiB blocks; what
    // does not divide is left unused
    if (op->slot_bytes % kBlockMsg) return MINT_ERR_GEOMETRY;
    a.step_blocks = op->slot_bytes / kBlockMsg / (uint32_t)a.shares;
    if (a.step_blocks == 0) return MINT_ERR_GEOMETRY;
    a.step_msg = a.step_blocks * kBlockMsg;
    if (op->waves_per_channel_group == 0 || a.step_blocks % op->waves_per_channel_group)
        return MINT_ERR_GEOMETRY;
    a.waves = (int)op->waves_per_channel_group;
    a.k_per_wave = a.step_blocks / (uint32_t)a.waves;
    const uint32_t raw_per_block = op->protocol == MINT_PROTO_LL128 ? kBlockRawLL : kBlockRawSimple;
    const uint64_t nblocks = (a.row_bytes + raw_per_block - 1) / raw_per_block;
    if (nblocks >= (1ull << 28)) return MINT_ERR_TOO_LARGE;
    a.nblocks = (uint32_t)nblocks;
    a.steps = (a.nblocks + a.step_blocks - 1) / a.step_blocks;
    if (a.steps > kMaxSteps) return MINT_ERR_TOO_LARGE;
    // (the temporal allgather numbers its steps through all rows)
    if (temporal && (uint64_t)a.steps * (uint64_t)op->world > kMaxSteps) return MINT_ERR_TOO_LARGE;
    a.credit_off = a.nslots * a.slot_bytes;
    if (op->credit_offset) {
        if (op->credit_offset < a.credit_off || op->credit_offset % 256) return MINT_ERR_GEOMETRY;
        a.credit_off = op->credit_offset;
    }
    a.epoch = op->flag_epoch;
    a.epoch_word = reinterpret_cast<const uint32_t*>(op->epoch_ptr);
    a.spin_budget = op->spin_budget ? op->spin_budget : kDefaultSpinBudget;
    a.status = reinterpret_cast<uint64_t*>(op->status);
    a.skip_origin = dbg ? dbg->skip_origin : 0u;
#ifdef MINT_RING_STATS
    a.stats = dbg ? reinterpret_cast<uint64_t*>(dbg->stats) : nullptr;
#else
    if (dbg && dbg->stats) return MINT_ERR_ARG;   // this build does not collect wait accounting
    a.stats = nullptr;
#endif
    a.placement = op->placement;
    {
        const int npos = a.hops + 1;
        a.seat_turn = (over_tree(op->op) || temporal) && kCusPerXcd % npos == 0
                          ? (uint32_t)(kCusPerXcd / npos) : 0u;
    }

    const int waves_per_block = (int)op->threads_per_block / 64;
    plan->threads = (int)op->threads_per_block;
    // Own rows through LDS: LL128 reductions, thread blocks of 4 or 7
    // wave-channels (plus the fetcher), one or two blocks per wave-channel and
    // step.  Everything else runs the walk that fetches its rows itself.
    a.k_per_wave = a.step_blocks / (uint32_t)a.waves;
    plan->lds = op->row_fetch == MINT_FETCH_LDS && op->protocol == MINT_PROTO_LL128 &&
                reducing(op->op) && !over_tree(op->op) &&
                (waves_per_block == 4 || waves_per_block == 7) &&
                a.k_per_wave % 4 != 0;
    a.fetch_depth = plan->lds ? kFetchDepth : 0u;
    if (!plan->lds && a.waves < waves_per_block) plan->threads = a.waves * 64;
    a.blocks_per_group = (a.waves * 64 + plan->threads - 1) / plan->threads;
    plan->blocks = a.pipes * (a.hops + 1) * a.blocks_per_group;
    // the XCD-local mapping deals whole channels to XCDs
    if (op->placement == MINT_PLACE_LOCAL && (a.pipes * a.blocks_per_group) % kXcds)
        return MINT_ERR_GEOMETRY;
    // Large sendrecvs, ring broadcasts, allgathers and alltoalls under the local placement: origins
    // on CUs which they have to themselves, as many as the caller names
    // (take_seat); the grid grows by the blocks that find nothing to do.
    a.origin_cus = 0;
    {
        const int npos = a.hops + 1, groups = a.pipes * a.blocks_per_group / kXcds;
        const int origin_cus = (int)op->origin_cus;
        if (origin_cus >= kCusPerXcd || op->reserved1) return MINT_ERR_ARG;
        plan->blocks_plain = plan->blocks;
        // (not for a launch so short that its seats are taken in the order of
        // arrival: there the list's order does not decide what a compute unit holds)
        const uint32_t walk_steps = temporal ? a.steps * (uint32_t)op->world : a.steps;
        if (op->placement == MINT_PLACE_LOCAL && origin_cus > 0 && npos >= 2 && groups >= 8 &&
            walk_steps >= kSeatByCuMinSteps &&
            (op->op == MINT_OP_BROADCAST || op->op == MINT_OP_ALLGATHER ||
             op->op == MINT_OP_SENDRECV || op->op == MINT_OP_ALLTOALL || temporal ||
             op->op == MINT_OP_TREE_BROADCAST)) {
            const int others = kCusPerXcd - origin_cus;
            const int r0 = (groups + origin_cus - 1) / origin_cus;
            const int r1 = ((npos - 1) * groups + others - 1) / others;
            a.origin_cus = (uint32_t)origin_cus;
            plan->blocks = kXcds * kCusPerXcd * (r0 > r1 ? r0 : r1);
        }
    }
    // (the map through which blocks claim their seats holds 1024 entries per XCD:
    // more thread blocks than a device keeps resident)
    if (op->placement == MINT_PLACE_LOCAL && plan->blocks / kXcds > kSeatWords * 64)
        return MINT_ERR_RESIDENCY;
    plan->unroll = a.k_per_wave % 4 == 0 ? 4 : (a.k_per_wave % 2 == 0 ? 2 : 1);
    // Every rank's staging ends in room for the counters the blocks of a launch
    // under the local placement claim their seats through (those of the first
    // rank that has staging are used): at the end of what the caller
    // allocated, so that launches of any geometry on the same staging find
    // the same counters, never another launch's credit words.
    const size_t credit_end = (size_t)a.credit_off + (size_t)a.shares * (size_t)a.waves * kCreditStride;
    plan->staging_need = credit_end + kTicketBytes;
    a.tickets = nullptr;
    {
        const size_t have = op->staging_bytes >= plan->staging_need ? (size_t)op->staging_bytes
                                                                    : plan->staging_need;
        const size_t ticket_off = (have - kTicketBytes) / 256 * 256;
        for (int r = 0; r < op->world && !a.tickets; ++r)
            if (op->staging[r]) a.tickets = reinterpret_cast<uint64_t*>(op->staging[r] + ticket_off);
    }
    if (op->placement == MINT_PLACE_LOCAL && !plan->empty && !a.tickets) return MINT_ERR_ARG;
    // The credit words lie behind the slots: a buffer that only holds the
    // slots (the reference's recvbuff is BUFF_SIZE bytes, 7_reducescatter.py:93)
    // would be written out of bounds.
    if (for_launch && !plan->empty && op->staging_bytes < plan->staging_need)
        return MINT_ERR_STAGING;
    return MINT_OK;
}

// The ring kernels are compiled one element type per translation unit
// (ring_family.hip), so that the build can run them side by side.
int launch_ring(const Plan& plan, int protocol, int dtype, int cache_policy, hipStream_t stream) {
    // the copying collectives move bytes whatever element type the caller names
    if (!reducing(plan.args.op)) dtype = MINT_BYTES;
    switch (dtype) {
        case MINT_F16: return launch_ring_family_f16(plan, protocol, cache_policy, stream);
        case MINT_BF16: return launch_ring_family_bf16(plan, protocol, cache_policy, stream);
        case MINT_F32: return launch_ring_family_f32(plan, protocol, cache_policy, stream);
        default: return launch_ring_family_bytes(plan, protocol, cache_policy, stream);
    }
}

// ---- the launch that allocates nothing ---------------------------------------
constexpr int kMaxDevices = 64;
constexpr size_t kStaticHeader = MINT_STATIC_HEADER_BYTES;
constexpr size_t kStaticRank = MINT_STATIC_RANK_BYTES;
constexpr size_t kStaticSlots = MINT_STATIC_SLOT_BYTES;
static_assert(kStaticRank % 256 == 0 && kStaticSlots % 256 == 0, "credit words are 256-byte lines");
static_assert(kStaticSlots + MINT_STATIC_CHANNELS * 256u + kTicketBytes <= kStaticRank, "seat tickets");
static_assert(kStaticHeader + MINT_MAX_RANKS * kStaticRank <= MINT_STATIC_SCRATCH_BYTES, "layout");

struct StaticScratch {
    std::atomic<unsigned char*> ptr{nullptr};   // device address of `scratch` on this device
};
StaticScratch g_static[kMaxDevices];

// Device address of this device's copy of `scratch` (looked up on the first
// call with that device current; `may_look_up` = false refuses instead: a
// stream under capture is no place for the look-up).
int static_scratch(unsigned char** out, bool may_look_up = true) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return MINT_ERR_HIP;
    if (dev < 0 || dev >= kMaxDevices) return MINT_ERR_ARG;
    unsigned char* p = g_static[dev].ptr.load(std::memory_order_acquire);
    if (!p) {
        if (!may_look_up) return MINT_ERR_NOT_READY;
        void* q = nullptr;
        if (hipGetSymbolAddress(&q, HIP_SYMBOL(scratch)) != hipSuccess || !q) {
            (void)hipGetLastError();
            return MINT_ERR_HIP;
        }
        p = static_cast<unsigned char*>(q);
        g_static[dev].ptr.store(p, std::memory_order_release);
    }
    *out = p;
    return MINT_OK;
}

template <int U>
int list_schedule(const RingArgs& a, uint32_t raw_per_block, int pipeline, int position, int wave,
                  uint32_t max_entries, uint32_t* step, uint32_t* block, uint32_t* recv_offset,
                  uint32_t* send_offset, uint32_t* n_entries) {
    uint64_t row_bytes;
    uint32_t nblocks, nfull;
    row_extent(a, pipeline, raw_per_block, row_bytes, nblocks, nfull);
    const WalkGeom geom{(uint32_t)a.waves, a.k_per_wave, a.step_blocks, a.nslots, a.slot_bytes,
                        a.step_msg, nblocks, nfull, (uint32_t)wave};
    const uint32_t share_recv = share_of(a, pipeline, position);
    const uint32_t share_send = share_of(a, pipeline, position + 1);
    const uint32_t ngroups = a.steps * (a.k_per_wave / (uint32_t)U);
    uint32_t n = 0;
    Group<U> q = Group<U>::first_of(geom);
    for (uint32_t i = 0; i < ngroups; ++i, q = q.next(geom)) {
        for (int u = 0; u < U; ++u) {
            if (!q.valid[u]) continue;
            if (n < max_entries) {
                if (step) step[n] = q.step;
                if (block) block[n] = q.g[u];
                if (recv_offset) recv_offset[n] = q.msg_off(geom, share_recv, u);
                if (send_offset) send_offset[n] = q.msg_off(geom, share_send, u);
            }
            ++n;
        }
    }
    *n_entries = n;
    return MINT_OK;
}

}  // namespace

extern "C" {

int mint_version(void) { return kVersion; }

int mint_build_flags(void) { return kBuildFlags; }

const char* mint_strerror(int err) {
    switch (err) {
        case MINT_OK: return "ok";
        case MINT_ERR_ARG: return "bad argument";
        case MINT_ERR_ALIGN: return "address not 16-byte aligned";
        case MINT_ERR_GEOMETRY: return "slot / wave geometry does not divide";
        case MINT_ERR_RESIDENCY: return "grid would not be co-resident on the device";
        case MINT_ERR_HIP: return "HIP runtime call failed";
        case MINT_ERR_TOO_LARGE: return "size does not fit the kernel's 32-bit counters";
        case MINT_ERR_STAGING: return "staging_bytes is smaller than mint_ring_staging_bytes()";
        case MINT_ERR_NOT_READY:
            return "first use on this device under stream capture: call mint_static_init() before";
        default: return "unknown error";
    }
}

int mint_device_info(int* compute_units, int* xcds, int* wave_size) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return MINT_ERR_HIP;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return MINT_ERR_HIP;
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (wave_size) *wave_size = prop.warpSize;
    if (xcds) {
        // Blocks are dealt round-robin over the XCDs: read the XCC_ID of the
        // first 64 blocks and count the distinct values.
        uint32_t* d = nullptr;
        if (hipMalloc(&d, 64 * sizeof(uint32_t)) != hipSuccess) return MINT_ERR_HIP;
        hipLaunchKernelGGL(xcd_map_kernel, dim3(64), dim3(64), 0, nullptr, d);
        uint32_t h[64];
        hipError_t e = hipMemcpy(h, d, sizeof(h), hipMemcpyDeviceToHost);
        (void)hipFree(d);
        if (e != hipSuccess) return MINT_ERR_HIP;
        uint32_t mask = 0;
        for (uint32_t v : h) mask |= 1u << (v & 31u);
        *xcds = __builtin_popcount(mask);
        // MINT_PLACE_LOCAL relies on more than the count: every aligned group
        // of 8 consecutive blocks has to land on 8 different XCDs.  Where the
        // probe does not show that, the device is reported as not dealing
        // regularly (0) and callers stay with MINT_PLACE_SPREAD.
        if (*xcds == kXcds) {
            for (int g = 0; g < 64; g += kXcds) {
                uint32_t seen = 0;
                for (int i = 0; i < kXcds; ++i) seen |= 1u << (h[g + i] & 31u);
                if (__builtin_popcount(seen) != kXcds) *xcds = 0;
            }
        }
    }
    return MINT_OK;
}

int mint_xcd_map(int blocks, void* out, void* stream) {
    if (blocks <= 0 || !out) return MINT_ERR_ARG;
    hipLaunchKernelGGL(xcd_map_kernel, dim3((unsigned)blocks), dim3(64), 0, as_stream(stream),
                       static_cast<uint32_t*>(out));
    return launch_status();
}

int mint_copy_simple(const void* src, void* dst, size_t nbytes, int blocks, int threads,
                     void* stream) {
    if (nbytes == 0) return MINT_OK;
    if (!src || !dst) return MINT_ERR_ARG;
    if (!aligned16(src) || !aligned16(dst)) return MINT_ERR_ALIGN;
    if (threads <= 0) threads = 512;
    if (threads % 64 || threads > 1024) return MINT_ERR_ARG;
    if (blocks <= 0) {
        blocks = device_cus() * (2048 / threads);
        if (blocks <= 0) return MINT_ERR_HIP;
    }
    const uint64_t need = (nbytes / 16 + (uint64_t)threads - 1) / (uint64_t)threads;
    if ((uint64_t)blocks > need) blocks = need ? (int)need : 1;
    hipLaunchKernelGGL(copy_simple_kernel, dim3((unsigned)blocks), dim3((unsigned)threads), 0,
                       as_stream(stream), static_cast<const uint8_t*>(src),
                       static_cast<uint8_t*>(dst), (uint64_t)nbytes);
    return launch_status();
}

int mint_read_xor(const void* src, size_t nbytes, void* out, int blocks, int threads,
                  void* stream) {
    if (!out) return MINT_ERR_ARG;
    if (nbytes < 16) return MINT_OK;
    if (!src) return MINT_ERR_ARG;
    if (!aligned16(src)) return MINT_ERR_ALIGN;
    if (threads <= 0) threads = 512;
    if (threads % 64 || threads > 1024) return MINT_ERR_ARG;
    if (blocks <= 0) {
        blocks = device_cus() * (2048 / threads);
        if (blocks <= 0) return MINT_ERR_HIP;
    }
    const uint64_t need = (nbytes / 16 + (uint64_t)threads - 1) / (uint64_t)threads;
    if ((uint64_t)blocks > need) blocks = (int)need;
    hipLaunchKernelGGL(read_xor_kernel, dim3((unsigned)blocks), dim3((unsigned)threads), 0,
                       as_stream(stream), static_cast<const uint8_t*>(src), (uint64_t)nbytes,
                       static_cast<uint32_t*>(out));
    return launch_status();
}

int mint_step_mix(const void* rows, size_t rows_bytes, void* staging, size_t staging_bytes,
                  int waves, int iters, int what, void* sink, void* stream) {
    if (waves <= 0 || iters <= 0 || what < 1 || (what & 9) == 8) return MINT_ERR_ARG;
    if ((what & 17) && (!rows || rows_bytes < (size_t)waves * (size_t)iters * kBlockRawLL))
        return MINT_ERR_ARG;
    if ((size_t)waves * (size_t)iters >= (1ull << 32)) return MINT_ERR_TOO_LARGE;
    if ((what & 6) && (!staging || staging_bytes < (size_t)waves * 2u * kBlockMsg)) return MINT_ERR_ARG;
    if ((what & 6) && staging_bytes >= (1ull << 31)) return MINT_ERR_TOO_LARGE;
    if ((what & 6) && !aligned16(staging)) return MINT_ERR_ALIGN;
    if (!(what & 20) && !sink) return MINT_ERR_ARG;
    void (*kernel)(const uint8_t*, uint8_t*, uint32_t, uint32_t, uint32_t, uint32_t*) = nullptr;
    switch (what) {
        case 1: kernel = step_mix_kernel<1>; break;
        case 2: kernel = step_mix_kernel<2>; break;
        case 3: kernel = step_mix_kernel<3>; break;
        case 4: kernel = step_mix_kernel<4>; break;
        case 5: kernel = step_mix_kernel<5>; break;
        case 6: kernel = step_mix_kernel<6>; break;
        case 7: kernel = step_mix_kernel<7>; break;
        case 9: kernel = step_mix_kernel<9>; break;
        case 11: kernel = step_mix_kernel<11>; break;
        case 13: kernel = step_mix_kernel<13>; break;
        case 15: kernel = step_mix_kernel<15>; break;
        case 16: kernel = step_mix_kernel<16>; break;
        case 18: kernel = step_mix_kernel<18>; break;
        case 20: kernel = step_mix_kernel<20>; break;
        case 22: kernel = step_mix_kernel<22>; break;
        case 7 + 2 * 256: kernel = step_mix_kernel<7 + 2 * 256>; break;
        case 7 + 4 * 256: kernel = step_mix_kernel<7 + 4 * 256>; break;
        case 7 + 5 * 256: kernel = step_mix_kernel<7 + 5 * 256>; break;
        case 7 + 6 * 256: kernel = step_mix_kernel<7 + 6 * 256>; break;
        case 7 + 8 * 256: kernel = step_mix_kernel<7 + 8 * 256>; break;
        case 7 + 12 * 256: kernel = step_mix_kernel<7 + 12 * 256>; break;
        default: return MINT_ERR_ARG;
    }
    const unsigned blocks = ((unsigned)waves + 3u) / 4u;
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(256), 0, as_stream(stream),
                       static_cast<const uint8_t*>(rows), static_cast<uint8_t*>(staging),
                       (uint32_t)staging_bytes, (uint32_t)waves, (uint32_t)iters,
                       static_cast<uint32_t*>(sink));
    return launch_status();
}

int mint_step_mix_deep(const void* rows, size_t rows_bytes, void* staging, size_t staging_bytes,
                       int waves, int iters, int what, int ahead, int partner, void* sink,
                       void* stream) {
    if (waves <= 0 || iters <= 0 || what < 1 || what > 7 || ahead < 1 || ahead > 3)
        return MINT_ERR_ARG;
    if (iters % (ahead + 1)) return MINT_ERR_ARG;          // whole rounds of the unrolled loop
    if ((what & 1) && (!rows || rows_bytes < (size_t)waves * (size_t)iters * kBlockRawLL))
        return MINT_ERR_ARG;
    if ((size_t)waves * (size_t)iters >= (1ull << 32)) return MINT_ERR_TOO_LARGE;
    const size_t need = (size_t)waves * (size_t)(ahead + 2) * kBlockMsg;
    if ((what & 6) && (!staging || staging_bytes < need)) return MINT_ERR_ARG;
    if ((what & 6) && staging_bytes >= (1ull << 31)) return MINT_ERR_TOO_LARGE;
    if ((what & 6) && !aligned16(staging)) return MINT_ERR_ALIGN;
    if (!(what & 4) && !sink) return MINT_ERR_ARG;
    using Kernel = void (*)(const uint8_t*, uint8_t*, uint32_t, uint32_t, uint32_t, uint32_t,
                            uint32_t*);
#define MINT_DEEP_ROW(A)                                                                        \
    {step_mix_deep_kernel<1, A>, step_mix_deep_kernel<2, A>, step_mix_deep_kernel<3, A>,        \
     step_mix_deep_kernel<4, A>, step_mix_deep_kernel<5, A>, step_mix_deep_kernel<6, A>,        \
     step_mix_deep_kernel<7, A>}
    static const Kernel table[3][7] = {MINT_DEEP_ROW(1), MINT_DEEP_ROW(2), MINT_DEEP_ROW(3)};
#undef MINT_DEEP_ROW
    const unsigned blocks = ((unsigned)waves + 3u) / 4u;
    hipLaunchKernelGGL(table[ahead - 1][what - 1], dim3(blocks), dim3(256), 0, as_stream(stream),
                       static_cast<const uint8_t*>(rows), static_cast<uint8_t*>(staging),
                       (uint32_t)staging_bytes, (uint32_t)waves, (uint32_t)iters, partner ? 1u : 0u,
                       static_cast<uint32_t*>(sink));
    return launch_status();
}

size_t mint_ll128_packed_bytes(size_t nbytes, int layout) {
    if (layout == MINT_LAYOUT_PAIR) return (nbytes + 119) / 120 * 128;
    return (nbytes + 959) / 960 * 1024;
}

int mint_ll128_pack(const void* raw, void* msg, size_t nbytes, uint64_t flag_base,
                    uint64_t flag_stride, int layout, void* stream) {
    if (layout != MINT_LAYOUT_PAIR && layout != MINT_LAYOUT_WAVE64) return MINT_ERR_ARG;
    if (nbytes == 0) return MINT_OK;
    if (!raw || !msg) return MINT_ERR_ARG;
    if (!aligned16(raw) || !aligned16(msg)) return MINT_ERR_ALIGN;
    const uint64_t lines = mint_ll128_packed_bytes(nbytes, layout) / 128;
    if (lines >= (1ull << 31)) return MINT_ERR_TOO_LARGE;
    const uint64_t waves = layout == MINT_LAYOUT_WAVE64 ? lines / 8 : (lines * 8 + 63) / 64;
    uint64_t blocks = (waves + 3) / 4;
    const uint64_t cap = (uint64_t)device_cus() * 8;
    if (cap && blocks > cap) blocks = cap;
    if (layout == MINT_LAYOUT_WAVE64)
        hipLaunchKernelGGL(pack_wave64_kernel, dim3((unsigned)blocks), dim3(256), 0,
                           as_stream(stream), static_cast<const uint8_t*>(raw),
                           static_cast<uint8_t*>(msg), (uint64_t)nbytes, (uint32_t)(lines / 8),
                           flag_base, flag_stride);
    else
        hipLaunchKernelGGL(pack_pair_kernel, dim3((unsigned)blocks), dim3(256), 0,
                           as_stream(stream), static_cast<const uint8_t*>(raw),
                           static_cast<uint8_t*>(msg), (uint64_t)nbytes, lines, flag_base,
                           flag_stride);
    return launch_status();
}

int mint_ll128_unpack(const void* msg, void* raw, size_t nbytes, uint64_t flag_base,
                      uint64_t flag_stride, int layout, void* bad_flags, void* stream) {
    if (layout != MINT_LAYOUT_PAIR && layout != MINT_LAYOUT_WAVE64) return MINT_ERR_ARG;
    if (nbytes == 0) return MINT_OK;
    if (!raw || !msg) return MINT_ERR_ARG;
    if (!aligned16(raw) || !aligned16(msg)) return MINT_ERR_ALIGN;
    const uint64_t lines = mint_ll128_packed_bytes(nbytes, layout) / 128;
    if (lines >= (1ull << 31)) return MINT_ERR_TOO_LARGE;
    const uint64_t waves = layout == MINT_LAYOUT_WAVE64 ? lines / 8 : (lines * 8 + 63) / 64;
    uint64_t blocks = (waves + 3) / 4;
    const uint64_t cap = (uint64_t)device_cus() * 8;
    if (cap && blocks > cap) blocks = cap;
    if (layout == MINT_LAYOUT_WAVE64)
        hipLaunchKernelGGL(unpack_wave64_kernel, dim3((unsigned)blocks), dim3(256), 0,
                           as_stream(stream), static_cast<const uint8_t*>(msg),
                           static_cast<uint8_t*>(raw), (uint64_t)nbytes, (uint32_t)(lines / 8),
                           flag_base, flag_stride, static_cast<unsigned long long*>(bad_flags));
    else
        hipLaunchKernelGGL(unpack_pair_kernel, dim3((unsigned)blocks), dim3(256), 0,
                           as_stream(stream), static_cast<const uint8_t*>(msg),
                           static_cast<uint8_t*>(raw), (uint64_t)nbytes, lines, flag_base,
                           flag_stride, static_cast<unsigned long long*>(bad_flags));
    return launch_status();
}

int mint_elementwise_sum(const void* a, const void* b, void* out, size_t nelem, int dtype,
                         void* stream) {
    if (dtype < MINT_F16 || dtype > MINT_F32) return MINT_ERR_ARG;
    if (nelem == 0) return MINT_OK;
    if (!a || !b || !out) return MINT_ERR_ARG;
    if (!aligned16(a) || !aligned16(b) || !aligned16(out)) return MINT_ERR_ALIGN;
    const uint64_t nbytes = (uint64_t)nelem * (dtype == MINT_F32 ? 4u : 2u);
    uint64_t blocks = (nbytes / 16 + 255) / 256;
    const uint64_t cap = (uint64_t)device_cus() * 8;
    if (blocks == 0) blocks = 1;
    if (cap && blocks > cap) blocks = cap;
    const uint8_t* pa = static_cast<const uint8_t*>(a);
    const uint8_t* pb = static_cast<const uint8_t*>(b);
    uint8_t* po = static_cast<uint8_t*>(out);
    switch (dtype) {
        case MINT_F16:
            hipLaunchKernelGGL(sum_kernel<DT_F16>, dim3((unsigned)blocks), dim3(256), 0,
                               as_stream(stream), pa, pb, po, nbytes);
            break;
        case MINT_BF16:
            hipLaunchKernelGGL(sum_kernel<DT_BF16>, dim3((unsigned)blocks), dim3(256), 0,
                               as_stream(stream), pa, pb, po, nbytes);
            break;
        default:
            hipLaunchKernelGGL(sum_kernel<DT_F32>, dim3((unsigned)blocks), dim3(256), 0,
                               as_stream(stream), pa, pb, po, nbytes);
    }
    return launch_status();
}

size_t mint_ring_staging_bytes(const mint_ring_op* op) {
    if (!op) return 0;
    // asked before the staging exists: absent addresses do not matter here
    mint_ring_op d = *op;
    for (int r = 0; r < MINT_MAX_RANKS; ++r)
        if (!d.staging[r]) d.staging[r] = 16;
    Plan plan;
    if (make_plan(&d, &plan) != MINT_OK) return 0;
    return plan.staging_need;
}

int mint_ring_grid_blocks(const mint_ring_op* op) {
    Plan plan;
    const int err = make_plan(op, &plan);
    return err != MINT_OK ? err : plan.blocks;
}

int mint_ring_schedule(const mint_ring_op* op, int pipeline, int position, int wave,
                       uint32_t max_entries, uint32_t* step, uint32_t* block,
                       uint32_t* recv_offset, uint32_t* send_offset, uint32_t* n_entries) {
    if (!n_entries) return MINT_ERR_ARG;
    *n_entries = 0;
    Plan plan;
    const int err = make_plan(op, &plan);
    if (err != MINT_OK) return err;
    if (plan.empty) return MINT_OK;
    if (over_tree(op->op) || over_hypercube(op->op) || op->op == MINT_OP_ALLGATHER_TEMPORAL)
        return MINT_ERR_ARG;                        // listed for the ring walks only
    const RingArgs& a = plan.args;
    if (pipeline < 0 || pipeline >= a.pipes || position < 0 || position > a.hops || wave < 0 ||
        wave >= a.waves)
        return MINT_ERR_ARG;
    const uint32_t raw = op->protocol == MINT_PROTO_LL128 ? kBlockRawLL : kBlockRawSimple;
    switch (plan.unroll) {
        case 4: return list_schedule<4>(a, raw, pipeline, position, wave, max_entries, step, block,
                                        recv_offset, send_offset, n_entries);
        case 2: return list_schedule<2>(a, raw, pipeline, position, wave, max_entries, step, block,
                                        recv_offset, send_offset, n_entries);
        default: return list_schedule<1>(a, raw, pipeline, position, wave, max_entries, step, block,
                                         recv_offset, send_offset, n_entries);
    }
}

int mint_ring_seat(const mint_ring_op* op, int xcd, int cu_rank, int nth, uint64_t* state,
                   int* pipeline, int* position, int* block_of_group) {
    Plan plan;
    const int err = make_plan(op, &plan);
    if (err != MINT_OK) return err;
    if (plan.empty || op->placement != MINT_PLACE_LOCAL || xcd < 0 || xcd >= kXcds || cu_rank < 0 ||
        nth < 0 || !state)
        return MINT_ERR_ARG;
    const SeatList list = seat_list(plan.args, plan.blocks);
    uint64_t* const taken = state;
    uint64_t& tickets = state[kSeatWords];
    int y;
    bool filled = false;
    if (seats_in_order_of_arrival(plan.args, list)) {
        // taken in the order of arrival at one counter per XCD
        y = tickets < (uint64_t)list.len ? (int)tickets : -1;
        ++tickets;
    } else {
        y = seat_claim(
            list, seat_wanted(list, cu_rank, nth),
            [&](int word, uint64_t bits) {
                const uint64_t before = taken[word];
                taken[word] |= bits;
                return before;
            },
            [&]() { return (int)tickets++; }, filled);
    }
    int p = 0, h = 0, gw = 0;
    if (y < 0 || !seat_of_entry(plan.args, xcd, y, p, h, gw)) return 0;
    if (pipeline) *pipeline = p;
    if (position) *position = h;
    if (block_of_group) *block_of_group = gw;
    return 1;
}

int mint_ring_launch(const mint_ring_op* op, void* stream) {
    return mint_ring_launch_debug(op, nullptr, stream);
}

int mint_ring_launch_debug(const mint_ring_op* op, const mint_ring_debug* dbg, void* stream) {
    Plan plan;
    const int err = make_plan(op, &plan, true, dbg);
    if (err != MINT_OK) return err;
    if (plan.empty) return MINT_OK;
    return launch_ring(plan, op->protocol, op->dtype, op->cache_policy, as_stream(stream));
}

int mint_ring_launch_static(const mint_ring_op* op, void* stream) {
    if (!op) return MINT_ERR_ARG;
    // size limits first: they need no device
    if ((uint64_t)op->nslots * op->slot_bytes > kStaticSlots) return MINT_ERR_TOO_LARGE;
    mint_ring_op d = *op;
    d.credit_offset = (uint32_t)kStaticSlots;
    d.staging_bytes = kStaticRank;
    d.flag_epoch = 0;
    d.epoch_ptr = 16;                 // stand-in until the address is known: any aligned non-zero value
    for (int r = 0; r < MINT_MAX_RANKS; ++r) d.staging[r] = 16;
    Plan plan;
    int err = make_plan(&d, &plan, true);
    if (err == MINT_ERR_STAGING) return MINT_ERR_TOO_LARGE;    // more credit words than the array holds
    if (err != MINT_OK) return err;
    if (plan.empty) return MINT_OK;

    // The array's address is looked up once per device.  Not while `stream` is
    // being captured into a graph: the first call on a device then has to have
    // happened before (mint_static_init).
    hipStream_t s = as_stream(stream);
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &capturing) != hipSuccess) {
        (void)hipGetLastError();
        capturing = hipStreamCaptureStatusNone;
    }
    unsigned char* base = nullptr;     // device address; never the array's name
    err = static_scratch(&base, capturing == hipStreamCaptureStatusNone);
    if (err != MINT_OK) return err;
    for (int r = 0; r < MINT_MAX_RANKS; ++r)
        plan.args.staging[r] = reinterpret_cast<uint64_t>(base + kStaticHeader + r * kStaticRank);
    // (the seat tickets sit at the end of rank 0's part, as in make_plan)
    plan.args.tickets = reinterpret_cast<uint64_t*>(
        base + kStaticHeader + (reinterpret_cast<size_t>(plan.args.tickets) - 16));
    uint32_t* epoch_word = reinterpret_cast<uint32_t*>(base);
    plan.args.epoch_word = epoch_word;

    // The array keeps what the last call left in it.  The epoch in its first
    // word makes old sector tags and credit words meaningless to this launch;
    // the kernel that advances it clears the array on first use, whenever the
    // 12-bit count starts over, and when an LL128 launch follows a Simple one
    // (raw payload of a Simple launch could pass for LL128 tags).  It takes
    // that decision on the device from the protocol word beside the epoch, so
    // a captured launch decides anew at every replay; the clearing is a fill
    // by the kernel itself, not a memset node.
    hipLaunchKernelGGL(epoch_advance_kernel, dim3(1), dim3(1024), 0, s, epoch_word,
                       base + kStaticHeader, (uint64_t)(MINT_STATIC_SCRATCH_BYTES - kStaticHeader),
                       kMaxEpoch, 1u, (uint32_t)op->protocol);
    if ((err = launch_status()) != MINT_OK) return err;
    return launch_ring(plan, op->protocol, op->dtype, op->cache_policy, s);
}

int mint_static_init(void) {
    unsigned char* base = nullptr;
    return static_scratch(&base);
}

int mint_epoch_advance(void* epoch_word, void* staging, size_t staging_bytes, int protocol,
                       void* stream) {
    if (!epoch_word || (reinterpret_cast<uint64_t>(epoch_word) & 3u)) return MINT_ERR_ARG;
    if (protocol < -1 || protocol > MINT_PROTO_SIMPLE) return MINT_ERR_ARG;
    if (staging_bytes && (!staging || !aligned16(staging) || staging_bytes % 16)) return MINT_ERR_ALIGN;
    hipLaunchKernelGGL(epoch_advance_kernel, dim3(1), dim3(1024), 0, as_stream(stream),
                       static_cast<uint32_t*>(epoch_word), static_cast<uint8_t*>(staging),
                       (uint64_t)staging_bytes, kMaxEpoch, protocol >= 0 ? 1u : 0u,
                       protocol >= 0 ? (uint32_t)protocol : 0u);
    return launch_status();
}

int mint_torn_line_probe(void* staging, size_t staging_bytes, int pairs, int iters,
                         int cache_policy, int placement, int per_sector, uint32_t flag_epoch,
                         uint32_t spin_budget, void* counters, void* stream) {
    if (!staging || !counters || pairs <= 0 || iters <= 0 || iters > (int)kMaxSteps ||
        flag_epoch == 0 || flag_epoch > kMaxEpoch)
        return MINT_ERR_ARG;
    if (!aligned16(staging)) return MINT_ERR_ALIGN;
    if (cache_policy < 0 || cache_policy > 2) return MINT_ERR_ARG;
    if (cache_policy == 2 && placement != MINT_PLACE_LOCAL) return MINT_ERR_ARG;
    const size_t need = (size_t)pairs * (kProbeDepth * kBlockMsg + 128u);
    if (staging_bytes < need || need >= (1ull << 31)) return MINT_ERR_ARG;
    const int wpb = 4, pair_blocks = (pairs + wpb - 1) / wpb, blocks = 2 * pair_blocks;
    if (placement == MINT_PLACE_LOCAL && pair_blocks % kXcds) return MINT_ERR_GEOMETRY;
    auto kernel = cache_policy == 0   ? torn_probe_kernel<Policy<0>::LD, Policy<0>::ST>
                  : cache_policy == 1 ? torn_probe_kernel<Policy<1>::LD, Policy<1>::ST>
                                      : torn_probe_kernel<Policy<2>::LD, Policy<2>::ST>;
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 256, 0) != hipSuccess)
        return MINT_ERR_HIP;
    if (blocks > per_cu * device_cus()) return MINT_ERR_RESIDENCY;
    hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream),
                       static_cast<uint8_t*>(staging), (uint32_t)pairs, (uint32_t)iters, placement,
                       per_sector ? 1 : 0, flag_epoch, spin_budget ? spin_budget : kDefaultSpinBudget,
                       static_cast<unsigned long long*>(counters));
    return launch_status();
}

}  // extern "C"
