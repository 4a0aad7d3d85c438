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
// wavefronts, so nothing has to lag).  Allreduce is the same walk carried on:
// 2 * world - 1 positions, the first `world` add, the rest copy, and every
// position from the last adder on keeps the result.  Alltoall is world * world
// pipelines of two positions: pipeline s * world + d carries row d of rank s
// straight into row s of rank d (every pair of virtual ranks is linked).
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
#include <type_traits>

#include "protocol.hpp"

namespace mint {

enum : int { OP_SENDRECV = 0, OP_BROADCAST = 1, OP_REDUCE = 2, OP_ALLGATHER = 3,
             OP_REDUCESCATTER = 4, OP_ALLREDUCE = 5, OP_ALLTOALL = 6,
             // (walks of their own: tree.hpp, temporal.hpp, hypercube.hpp)
             OP_TREE_BROADCAST = 7, OP_TREE_REDUCE = 8, OP_ALLGATHER_TEMPORAL = 9,
             OP_HYPER_REDUCESCATTER = 10, OP_HYPER_ALLGATHER = 11 };
enum : int { PROTO_LL128 = 0, PROTO_SIMPLE = 1 };
enum : int { PLACE_SPREAD = 0, PLACE_LOCAL = 1 };

constexpr int kMaxRanks = 8;
constexpr int kXcds = 8;                  // XCDs of an MI355X; blocks are dealt over them round-robin
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
    uint64_t total_bytes;                 // 0, or clip row p to total_bytes - p * row_stride
    int32_t phases;                       // staging shares per pipeline (2 for allreduce)
    int32_t shares;                       // shares of a slot: pipes * phases; alltoall: one per source rank
    uint32_t nblocks;                     // blocks per row
    uint32_t steps;                       // steps per row
    uint32_t slot_bytes, nslots;
    uint32_t step_msg;                    // bytes of one share: slot_bytes / (pipes * phases)
    uint32_t step_blocks;                 // step_msg / 1024
    uint32_t k_per_wave;                  // step_blocks / waves
    uint32_t credit_off;                  // offset of the credit words in staging
    uint32_t epoch, spin_budget;
    const uint32_t* epoch_word;           // optional: take the epoch from device memory instead
    uint64_t* status;
    uint32_t skip_origin;
    uint32_t seat_turn;                   // local placement: channels after which the positions turn by two (0: never)
    uint32_t origin_cus;                  // local placement: of the 32 CUs of an XCD, so many hold origins only (0: the plain order)
    uint64_t* stats;                      // optional: per position 8 x u64 of wait accounting
    uint32_t fetch_depth;                 // own rows through LDS: groups of LDS per wave-channel
    uint64_t* tickets;                    // local placement: the words seats are claimed through (kTicket*)
};

struct Role {
    int rank, next;
    bool load, recv, reduce, save, send;
};

__device__ __forceinline__ Role role_of(const RingArgs& a, int p, int h) {
    Role r;
    if (a.op == OP_ALLTOALL) {
        // pipeline p = source * world + destination: origin, then sink
        const int src = p / a.world, dst = p % a.world;
        r.rank = h == 0 ? src : dst;
        r.next = dst;
        r.load = r.send = h == 0;
        r.recv = r.save = h != 0;
        r.reduce = false;
        return r;
    }
    const int s = a.start[p];
    r.rank = a.cyc[(s + h) % a.cyc_len];
    r.next = a.cyc[(s + h + 1) % a.cyc_len];
    const bool origin = h == 0, sink = h == a.hops;
    r.recv = !origin;
    r.send = !sink;
    if (a.op == OP_ALLREDUCE) {
        // reduce-scatter then all-gather in one pass around the ring: the
        // first `world` positions add (the last of them holds the finished
        // sum and keeps a copy), the rest copy and forward
        const bool adding = h < a.world;
        r.load = adding;
        r.reduce = adding && !origin;
        r.save = h >= a.world - 1;
        return r;
    }
    const bool reducing = a.op == OP_REDUCE || a.op == OP_REDUCESCATTER;
    const bool copying_all = a.op == OP_BROADCAST || a.op == OP_ALLGATHER;
    r.load = origin || (reducing && !sink);
    r.reduce = reducing && !origin && !sink;
    r.save = sink || (copying_all && !origin);
    return r;
}

// First wavefront that gives up records why (1 = a bounded wait ran out,
// 2 = the local placement met an XCD number beyond 7, 3 = no seat) and who
// it was; everybody else sees word 3: its low half is the abort flag, its
// high half counts the launches that started with the flag set.
__device__ __forceinline__ void report_error(uint64_t* status, uint64_t code, int p, int h, int w,
                                             uint64_t detail) {
    if (lane_id() == 0) {
        unsigned long long* s = reinterpret_cast<unsigned long long*>(status);
        if (atomicCAS(s, 0ull, (unsigned long long)code) == 0ull) {
            st64_agent(status + 1, ((uint64_t)p << 32) | ((uint64_t)h << 16) | (uint64_t)w);
            st64_agent(status + 2, detail);
        }
        __hip_atomic_fetch_or((MINT_GLOBAL unsigned long long*)(s + 3), 1ull, __ATOMIC_RELAXED,
                              __HIP_MEMORY_SCOPE_AGENT);
    }
}
__device__ __forceinline__ void report_timeout(uint64_t* status, int p, int h, int w,
                                               uint64_t step) {
    report_error(status, 1, p, h, w, step);
}
__device__ __forceinline__ bool aborted(const uint64_t* status) {
    return __builtin_amdgcn_readfirstlane((uint32_t)ld64_agent(status + 3)) != 0u;
}
// One wavefront per launch: a launch that starts with the abort flag set (an
// earlier launch on this status block gave up and the caller has not looked
// yet) gives up at its first wait; count it, so that the caller learns how
// many launches ran for nothing.
__device__ __forceinline__ void count_launch_if_aborted(uint64_t* status, int wave_of_block) {
    if (blockIdx.x == 0 && wave_of_block == 0 && lane_id() == 0 && aborted(status))
        __hip_atomic_fetch_add((MINT_GLOBAL unsigned long long*)(status + 3), 1ull << 32,
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Spin until the credit / head word at `word` carries this epoch and a count
// of at least `need`.  Returns false when the budget ran out or somebody
// aborted.  (wait_ll128, protocol.py:161-180, with a bound.)
__device__ __forceinline__ bool wait_count(const uint64_t* word, uint32_t epoch, uint32_t need,
                                           uint32_t& cached, uint32_t budget,
                                           const uint64_t* status) {
    if (cached >= need) return true;
    for (uint32_t spins = 0;; ++spins) {
        uint64_t v = ld64_agent(word);
        uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
        uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
        if (hi == epoch && lo >= need) { cached = lo; return true; }
        if (spins >= budget) return false;
        if ((spins & 63u) == 63u && aborted(status)) return false;
        __builtin_amdgcn_s_sleep(2);
    }
}

// Which (pipeline, position, wave-channel) a wavefront serves.  `wpb` =
// wave-channels per thread block, `wib` = this wavefront's index among them.
constexpr int kCusPerXcd = 32;      // MI355X: 256 CUs in 8 XCDs
struct Seat {
    int p, h, gw, w;
    bool ok;
};
__device__ __forceinline__ int seat_wave(const RingArgs& a, int gw, int wpb, int wib) {
    // Index of a wave-channel inside its group: it decides which blocks of
    // a step, which staging bytes and which credit word the wave owns.  Under
    // the local placement the blocks of one XCD are numbered consecutively, so
    // that what an XCD touches (staging, rows) is contiguous in memory instead
    // of 4 KiB out of every 32: that spreads it over all channels and sets of
    // that XCD's L2.
    if (a.placement == PLACE_LOCAL && a.blocks_per_group % kXcds == 0 && a.waves % wpb == 0)
        return (gw % kXcds) * (a.waves / kXcds) + (gw / kXcds) * wpb + wib;
    return gw * wpb + wib;
}

// ---- seats under the local placement --------------------------------------------
// XCD d serves the channels c with c % 8 == d: a channel's whole ring then
// shares one L2.  The work of an XCD is a list of entries; entry y is one
// (channel, position).  Which entry a thread block takes does not depend on
// its number: the block asks the hardware where it runs (XCC_ID, and the
// compute unit's number from HW_ID) and claims an entry through counters in
// device memory.  Every block gets an entry, and every entry goes to exactly
// one block, whatever way the device deals its blocks over the compute units
// of an XCD (a stream confined to some of them, compute units busy with
// another stream's kernel, a grid that is only partly resident at any time),
// provided every XCD receives an eighth of the grid; a block that finds its
// XCD's list taken ends the launch with status 3.
//
// The list of an XCD is walked in rounds of one entry per compute unit: the
// compute unit that was the j-th of its XCD to show up wants, with its n-th
// block, entry n * 32 + j.  All blocks of a compute unit so share j, and the
// order of the list decides what a compute unit holds: with h = y % npos and
// a position count that divides 32 (8 ranks) every compute unit holds blocks
// of one position only - the positions that load from HBM sit on compute
// units of their own and the polls of the others, answered by the L2, never
// queue behind a load from HBM in a compute unit's memory pipeline.  The ring
// walks are fastest that way (an allgather whose compute units hold a mix of
// positions takes 4 - 10 % longer; the order in which blocks reach a counter
// is nothing like the order of their numbers, so one counter per XCD would
// mix them).  An entry is claimed by setting its bit in the XCD's map of
// taken entries; a block that wants none (a last, partial round of a list
// that is no multiple of 32; a compute unit that got more than its share; a
// 33rd compute unit) or finds its entry taken draws a ticket: the first
// `rest` tickets start at their entry of the partial round, all later ones at
// the head of the list, and a block takes the first free entry from there
// upwards.  With every compute unit at its share that is one look at the
// partial round each; with any other deal the blocks sort themselves out - as
// many blocks as entries, so there is a free one for everybody - and only the
// neat division of positions over compute units is lost.  (From the head
// upwards, because a list is also the order in which channels become
// complete: where not all blocks are resident at once - half of the compute
// units masked off - the blocks that are there have to fill whole channels,
// lowest first, or they wait for blocks that cannot start.)
//
// The counters (64-bit words in device memory, zero at first; between
// launches zero again but for the compute units' ranks):
//   xcd * 2048 + cu * 8     per compute unit: blocks that have arrived in bits
//                           23:0, j + 1 in bits 31:24 once it is known (kept)
//   16384 + xcd * 128       per XCD, a line of its own: + 0 compute units
//                           registered (kept), + 8 tickets handed out, + 16 entries
//                           claimed (a list taken in the order of arrival) or
//                           words of the map that are full
//   18432 + xcd * 128       per XCD, a line of its own: the map of taken
//                           entries, 1024 bits
// A line that blocks of several XCDs work on is slow (a counter per XCD in one
// line: 40 - 60 us for 160 blocks per XCD; in lines of their own: 6 us), hence
// the spacing.  The block that claims the last entry of its XCD's list puts
// that XCD's counters back to zero, so a launch finds them as the launch
// before left them and the common path is one atomic per counter
// (with the launch epoch in every word instead, every block of a launch found
// a stale word first and went through a compare-and-swap: three more trips).
// Nothing waits for the whole grid to be seated: a launch whose blocks are
// not all resident at once (a stream confined to half of the compute units)
// runs the channels that are complete, and their blocks make room for the
// rest.  A launch that could not seat all its blocks (status 2 or 3) leaves
// counters behind: the staging is cleared before it is used again.  All of
// these are atomics and loads at agent scope: one place serves them whichever
// XCD asks.
constexpr uint32_t kTicketXcdLine = 16384, kTicketXcdStride = 128, kTicketTaken = 18432;
constexpr uint32_t kTicketBytes = 20 * 1024;
constexpr uint32_t kSeatPatience = 1u << 18;
constexpr int kSeatWords = 16;            // map of taken entries: 1024 per XCD at most

// The list of one XCD: `len` entries, of which the first `full` rounds are
// taken by (compute unit, arrival) and the `rest` after them by leftover ticket.
struct SeatList {
    int len, full, rest;
};
__host__ __device__ __forceinline__ SeatList seat_list(const RingArgs& a, int grid_blocks) {
    SeatList l;
    l.len = grid_blocks / kXcds;
    l.full = l.len / kCusPerXcd;
    l.rest = l.len % kCusPerXcd;
    return l;
}
// Entry the block that arrived `nth` on the compute unit registered as `j`-th
// of its XCD wants; -1: none, it draws a ticket.
__host__ __device__ __forceinline__ int seat_wanted(const SeatList& l, int j, int nth) {
    return j < kCusPerXcd && nth < l.full ? nth * kCusPerXcd + j : -1;
}
// Claims `wanted`, or - with -1 or the entry taken - a free entry by ticket:
// ticket t < rest starts at entry t of the partial round, every later one at
// entry 0, and takes the first free entry from there upwards (round the list).
// `fetch_or(word, bits)` sets bits in word `word` of the XCD's map of taken
// entries and returns what the word held before; `draw()` hands out the next
// ticket.  -1: no entry is free (more blocks than entries).  `filled_a_word`
// comes back true for the block whose claim set the last free entry of a word
// of the map: exactly one block per word learns that.
template <class FetchOr, class Draw>
__host__ __device__ __forceinline__ int seat_claim(const SeatList& l, int wanted, FetchOr fetch_or,
                                                   Draw draw, bool& filled_a_word) {
    const int last_word = (l.len - 1) >> 6;
    // bits of word `word` that stand for entries of the list
    auto entries_of = [&](int word) {
        return word == last_word && (l.len & 63) ? (1ull << (l.len & 63)) - 1ull : ~0ull;
    };
    filled_a_word = false;
    if (wanted >= 0) {
        const uint64_t bit = 1ull << (wanted & 63), before = fetch_or(wanted >> 6, bit);
        if (!(before & bit)) {
            filled_a_word = (before | bit) == entries_of(wanted >> 6);
            return wanted;
        }
    }
    const int t = draw();
    int e = t < l.rest ? l.full * kCusPerXcd + t : 0;
    // (every miss means that another block took an entry, so len looks and a
    // walk over the words suffice)
    for (int looks = 0; looks < l.len + 2 * kSeatWords; ++looks) {
        const int word = e >> 6, bit = e & 63;
        const uint64_t before = fetch_or(word, 1ull << bit);
        if (!((before >> bit) & 1ull)) {
            filled_a_word = (before | (1ull << bit)) == entries_of(word);
            return e;
        }
        // the lowest entry of this word above e that was free a moment ago
        const uint64_t free_above = ~before & ~((2ull << bit) - 1ull) & entries_of(word);
        if (free_above) e = word * 64 + __builtin_ctzll(free_above);
        else e = word < last_word ? (word + 1) * 64 : 0;
    }
    return -1;
}
// A list of at most one round (a small launch: no compute unit gets a second
// block) is simply taken in the order in which the blocks reach one counter:
// one trip to the counter instead of three or four in a row.  So is the list
// of a launch of fewer than kSeatByCuMinSteps steps, whose few microseconds
// gain more from the shorter start than from a neat division of the positions
// over the compute units (8 ranks, 1 - 4 MiB per rank: -1.5 us of 14 - 28; from
// 17 steps on the copying collectives, whose origins want compute units of
// their own, lose 20 % that way, and long reductions 5 - 8 %; a temporal
// allgather runs its steps once per rank).
constexpr uint32_t kSeatByCuMinSteps = 16;
__host__ __device__ __forceinline__ bool seats_in_order_of_arrival(const RingArgs& a,
                                                                   const SeatList& l) {
    const uint32_t steps = a.op == OP_ALLGATHER_TEMPORAL ? a.steps * (uint32_t)a.world : a.steps;
    return l.full == 0 || steps < kSeatByCuMinSteps;
}
// What entry y of XCD `xcd` is: pipeline, position, block of the group.
__host__ __device__ __forceinline__ bool seat_of_entry(const RingArgs& a, int xcd, int y, int& p,
                                                       int& h, int& gw) {
    const int npos = a.hops + 1;
    // seat_turn turns the positions by two after every round over the compute
    // units, which mixes them: the tree gains 10 % from that
    int q = y / npos;
    h = a.seat_turn ? (y % npos + (q / (int)a.seat_turn) * 2) % npos : y % npos;
    if (a.origin_cus) {
        // Origins on compute units of their own, and on more of them than
        // their share of the blocks: in every round origin_cus of the compute
        // units take an origin, the others take the receiving positions of the
        // channels in turn.  Entries left over in either list are empty.
        // (What a compute unit's memory pipeline keeps in flight is bounded;
        // loads from HBM under a collective's stores take 2.5 us, so a
        // compute unit full of origins delivers 10 GB/s and an eighth of them
        // cannot feed the rest: allgather 8 x 128 MiB 3.4 ms, 1.9 ms without
        // its loads.)
        const int round = y / kCusPerXcd, j = y % kCusPerXcd, o = (int)a.origin_cus;
        const int groups = a.pipes * a.blocks_per_group / kXcds;
        // the origins' compute units lie evenly among the 32: `before` of them below j
        const int before = j * o / kCusPerXcd;
        if ((j + 1) * o / kCusPerXcd > before) {
            q = round * o + before;
            h = 0;
        } else {
            const int r = round * (kCusPerXcd - o) + (j - before);
            q = r / (npos - 1);
            h = 1 + r % (npos - 1);
        }
        if (q >= groups) return false;
    }
    const int c = q * kXcds + xcd;
    p = c / a.blocks_per_group;
    gw = c % a.blocks_per_group;
    return true;
}

__device__ __forceinline__ uint32_t launch_epoch(const RingArgs& a) {
    // The epoch normally is a launch argument; a caller that replays captured
    // launches keeps it in device memory and advances it between launches.
    return a.epoch_word ? __builtin_amdgcn_readfirstlane(__hip_atomic_load(
                              as_global(a.epoch_word), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
                        : a.epoch;
}
__device__ __forceinline__ uint64_t* ticket_word(const RingArgs& a, uint32_t byte_offset) {
    return reinterpret_cast<uint64_t*>(reinterpret_cast<uint8_t*>(a.tickets) + byte_offset);
}
__device__ __forceinline__ uint64_t ticket_add(uint64_t* word, uint64_t v) {
    return __hip_atomic_fetch_add((MINT_GLOBAL unsigned long long*)word, (unsigned long long)v,
                                  __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// The entry of its XCD's list this thread block takes (called by one lane of
// the block), or -1.  `xcd` comes back as the XCD it runs on, `last` says that
// the block claimed the last entry of that XCD's list (it then puts the XCD's
// counters back to zero: reset_tickets).  The wait here is for another block to
// be dispatched, not for data: it gets at least kSeatPatience looks whatever
// budget the caller gave the data waits.
__device__ __forceinline__ int claim_entry(const RingArgs& a, int& xcd, bool& last) {
    last = false;
    xcd = xcc_id();
    if (xcd >= kXcds) {
        report_error(a.status, 2, 0, 0, 0, (uint64_t)xcd);
        return -1;
    }
    const SeatList list = seat_list(a, (int)gridDim.x);
    uint64_t* const line = ticket_word(a, kTicketXcdLine + (uint32_t)xcd * kTicketXcdStride);
    int y;
    uint32_t claimed = 0;
    if (seats_in_order_of_arrival(a, list)) {
        claimed = (uint32_t)ticket_add(line + 2, 1ull);
        y = (int)claimed < list.len ? (int)claimed : -1;
    } else {
        // compute unit number inside the XCD: HW_ID bits 15:8 (CU, SH, SE)
        const uint32_t cu = __builtin_amdgcn_s_getreg(4 | (8 << 6) | (7 << 11));
        uint64_t* const word = ticket_word(a, (uint32_t)xcd * 2048u + cu * 8u);
        const uint32_t before = (uint32_t)ticket_add(word, 1ull);
        const uint32_t nth = before & 0xFFFFFFu;
        uint32_t jfield = before >> 24;
        if (before == 0u) {
            // first block this compute unit ever ran on this staging: register
            // the unit, publish its j (which stays: later launches find it)
            jfield = (uint32_t)ticket_add(line, 1ull) + 1u;
            if (jfield > 0xFFu) jfield = 0xFFu;
            __hip_atomic_fetch_or((MINT_GLOBAL unsigned long long*)word,
                                  (unsigned long long)jfield << 24, __ATOMIC_RELAXED,
                                  __HIP_MEMORY_SCOPE_AGENT);
        } else {
            const uint32_t budget = a.spin_budget < kSeatPatience ? kSeatPatience : a.spin_budget;
            for (uint32_t spins = 0; jfield == 0u; ++spins) {
                if (spins >= budget) {
                    report_error(a.status, 3, 0, 0, 0, (uint64_t)cu);
                    return -1;
                }
                __builtin_amdgcn_s_sleep(1);
                jfield = ((uint32_t)ld64_agent(word) >> 24) & 0xFFu;
            }
            jfield &= 0xFFu;
        }
        uint64_t* const taken = ticket_word(a, kTicketTaken + (uint32_t)xcd * kTicketXcdStride);
        bool filled = false;
        y = seat_claim(
            list, seat_wanted(list, (int)jfield - 1, (int)nth),
            [&](int word, uint64_t bits) {
                return (uint64_t)__hip_atomic_fetch_or((MINT_GLOBAL unsigned long long*)(taken + word),
                                                       (unsigned long long)bits, __ATOMIC_RELAXED,
                                                       __HIP_MEMORY_SCOPE_AGENT);
            },
            [&]() { return (int)ticket_add(line + 1, 1ull); }, filled);
        if (y < 0) {
            report_error(a.status, 3, 0, 0, 0, (uint64_t)cu);
            return -1;
        }
        // The block that fills the last word of the map has claimed the last
        // entry of the list (words are counted as they fill up: one more trip
        // for 4 - 16 blocks per XCD instead of one for every block).
        const uint32_t words = (uint32_t)((list.len + 63) >> 6);
        last = filled && (uint32_t)ticket_add(line + 2, 1ull) + 1u == words;
        return y;
    }
    if (y < 0) return -1;
    // the block that claims the last entry of its XCD's list clears up
    last = claimed + 1u == (uint32_t)list.len;
    return y;
}
// Puts the counters of XCD `xcd` back for the next launch (the thread block
// that claimed the last entry of the XCD's list; every other claim of the
// launch on this XCD has been counted by then).  What stays is the compute
// units' ranks - the j of every unit that has registered and the count of
// those - so that from the second launch on a block reads its unit's j from
// the word it counts itself on, instead of registering the unit again (two
// trips fewer at the start of every launch, and nobody waits for a j).
__device__ __forceinline__ void reset_tickets(const RingArgs& a, int xcd) {
    for (uint32_t i = threadIdx.x; i < 256u + 2u + (uint32_t)kSeatWords; i += blockDim.x) {
        if (i < 256u) {
            __hip_atomic_fetch_and((MINT_GLOBAL unsigned long long*)ticket_word(a, (uint32_t)xcd * 2048u + i * 8u),
                                   0xFF000000ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            continue;
        }
        uint64_t* const w =
            i < 258u ? ticket_word(a, kTicketXcdLine + (uint32_t)xcd * kTicketXcdStride) + (i - 255u)
                     : ticket_word(a, kTicketTaken + (uint32_t)xcd * kTicketXcdStride) + (i - 258u);
        __hip_atomic_store((MINT_GLOBAL unsigned long long*)w, 0ull, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    }
}
// The seat of this wavefront.  Under the local placement wavefront 0 of the
// thread block claims the block's entry and hands it to the others through
// `shared_entry` (an int of LDS): every wavefront of the block has to call.
__device__ __forceinline__ Seat take_seat(const RingArgs& a, int wpb, int wib, int wave_of_block,
                                          MINT_LDS int* shared_entry) {
    // (locals, not members of the result: a member passed by reference keeps
    // the whole struct in scratch memory)
    int p = 0, h = 0, gw = 0;
    bool seated = true;
    count_launch_if_aborted(a.status, wave_of_block);
    if (a.placement == PLACE_LOCAL) {
        if (wave_of_block == 0 && lane_id() == 0) {       // one lane: the counters count blocks
            int xcd = 0;
            bool last = false;
            const int y = claim_entry(a, xcd, last);
            shared_entry[0] = y < 0 ? -1 : (y * kXcds + xcd) * 2 + (last ? 1 : 0);
        }
        __syncthreads();
        const int e = __builtin_amdgcn_readfirstlane(shared_entry[0]);
        if (e >= 0 && (e & 1)) reset_tickets(a, (e >> 1) % kXcds);
        seated = e >= 0 && seat_of_entry(a, (e >> 1) % kXcds, (e >> 1) / kXcds, p, h, gw);
    } else {
        const int npos = a.hops + 1, x = (int)blockIdx.x;
        const int c = x / npos;
        h = x % npos;
        p = c / a.blocks_per_group;
        gw = c % a.blocks_per_group;
    }
    Seat st;
    st.p = p; st.h = h; st.gw = gw; st.w = 0;
    st.ok = false;
    if (!seated || gw * wpb + wib >= a.waves) return st;
    st.w = seat_wave(a, gw, wpb, wib);
    st.ok = !(h == 0 && a.skip_origin);
    return st;
}

// ---- chunk scheduler --------------------------------------------------------
// Which blocks of its row a wave-channel moves, in which order, and where they
// sit in a staging slot (the reference computes this inline in every kernel,
// e.g. 7_reducescatter.py:23-34,43-44,75-77).  Host and device share this
// code: the kernels walk it, mint_ring_schedule lists it.
//
// A row is cut into blocks (960 raw bytes for LL128, 1024 for Simple).  Step s
// covers blocks [s * step_blocks, (s + 1) * step_blocks); inside a step,
// wave-channel w of W takes blocks k * W + w, k = 0 .. K - 1, U at a time (a
// group).  Block i of a step travels in bytes [i * 1024, (i + 1) * 1024) of
// this (pipeline, phase)'s share of slot s mod nslots.
struct WalkGeom {
    uint32_t waves, k_per_wave, step_blocks, nslots, slot_bytes, step_msg;
    uint32_t nblocks;        // blocks of this row (allreduce rows may be clipped)
    uint32_t nfull;          // of which lie wholly inside the row
    uint32_t w;              // this wave-channel
};
template <int U>
struct Group {
    uint32_t step, slot, k0, idx[U], g[U];
    bool valid[U], full[U], first, last;
    __host__ __device__ __forceinline__ void fill(const WalkGeom& s) {
        first = k0 == 0;
        last = k0 + (uint32_t)U >= s.k_per_wave;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            idx[u] = (k0 + (uint32_t)u) * s.waves + s.w;
            g[u] = step * s.step_blocks + idx[u];
            valid[u] = g[u] < s.nblocks;
            full[u] = g[u] < s.nfull;
        }
    }
    __host__ __device__ __forceinline__ static Group first_of(const WalkGeom& s) {
        Group q;
        q.step = 0; q.slot = 0; q.k0 = 0;
        q.fill(s);
        return q;
    }
    // The walk over (step, first block) is kept incrementally: no division.
    __host__ __device__ __forceinline__ Group next(const WalkGeom& s) const {
        Group q;
        q.step = step; q.slot = slot; q.k0 = k0 + (uint32_t)U;
        if (q.k0 >= s.k_per_wave) {
            q.k0 = 0;
            ++q.step;
            q.slot = slot + 1 == s.nslots ? 0 : slot + 1;
        }
        q.fill(s);
        return q;
    }
    // byte offset of block u of this group inside a rank's staging
    __host__ __device__ __forceinline__ uint32_t msg_off(const WalkGeom& s, uint32_t share,
                                                         int u) const {
        return slot * s.slot_bytes + share * s.step_msg + idx[u] * 1024u;
    }
};
// Row p of the launch: its length (allreduce splits one buffer into `world`
// rows; the last ones may be short or empty) and its block counts.
__host__ __device__ __forceinline__ void row_extent(const RingArgs& a, int p, uint32_t raw_per_block,
                                                    uint64_t& row_bytes, uint32_t& nblocks,
                                                    uint32_t& nfull) {
    const uint64_t row_off = (uint64_t)p * a.row_stride;
    row_bytes = a.row_bytes;
    nblocks = a.nblocks;
    if (a.total_bytes) {
        const uint64_t left = a.total_bytes > row_off ? a.total_bytes - row_off : 0;
        row_bytes = left < a.row_bytes ? left : a.row_bytes;
        nblocks = (uint32_t)((row_bytes + raw_per_block - 1) / raw_per_block);
    }
    nfull = (uint32_t)(row_bytes / raw_per_block);    // these take the unguarded path
}
// A rank can receive twice in one pipeline of an allreduce (once while the sum
// is built, once while it is handed round): each phase has its own share of
// the slots and its own credit words.
__host__ __device__ __forceinline__ uint32_t share_of(const RingArgs& a, int p, int h) {
    if (a.op == OP_ALLTOALL) return (uint32_t)(p / a.world);      // the source rank's share
    return (uint32_t)p * (uint32_t)a.phases + (h >= a.world && a.phases > 1 ? 1u : 0u);
}
// Rows of the caller's buffers a pipeline reads and writes: row p of every
// rank, except alltoall, where pipeline source * world + destination reads row
// `destination` of the source and writes row `source` of the destination.
__host__ __device__ __forceinline__ uint32_t row_read(const RingArgs& a, int p) {
    return a.op == OP_ALLTOALL ? (uint32_t)(p % a.world) : (uint32_t)p;
}
__host__ __device__ __forceinline__ uint32_t row_written(const RingArgs& a, int p) {
    return a.op == OP_ALLTOALL ? (uint32_t)(p / a.world) : (uint32_t)p;
}

// How staging memory is accessed.  The sector tags make any choice safe: a
// stale or partially visible sector fails its tag test and is polled again,
// so a wrong policy costs time (or a reported time-out), never data.
//   0  agent scope: loads and stores miss / write through the per-XCD L2, so
//      producer and consumer may sit on different XCDs
//   1  system scope
//   2  XCD-local: stores (and credit words) carry no scope bits and stay in
//      the L2 of the XCD; loads are agent scope, which skips the per-CU L1 and
//      is served by that L2 while the line is still there.  Only valid with
//      PLACE_LOCAL, where all hops of a channel share one XCD (each block
//      takes its work from the XCD it finds itself on).
//      (Measured alternatives: nt loads behave like sc1 loads; plain and sc0
//      loads keep hitting stale L1 lines and time out, with or without
//      buffer_inv sc0.)
template <int CPI> struct Policy;
template <> struct Policy<0> { static constexpr int LD = CP_SC1, ST = CP_SC1; };
template <> struct Policy<1> { static constexpr int LD = CP_SYSTEM, ST = CP_SYSTEM; };
template <> struct Policy<2> { static constexpr int LD = CP_SC1, ST = CP_NONE; };

// A role whose flags are compile-time constants.
template <bool LOAD, bool RECV, bool REDUCE, bool SAVE, bool SEND>
struct FixedRole {
    int rank, next;
    static constexpr bool load = LOAD, recv = RECV, reduce = REDUCE, save = SAVE, send = SEND;
};

// ---- own rows through LDS ------------------------------------------------------
// Vector-memory loads of one wavefront return in issue order, so a wave-channel
// that fetches its own rows from HBM itself has every poll of staging (an L2
// hit) queue behind the HBM fetch issued just before it: its step can never be
// shorter than an HBM round trip, however far ahead it fetches.  With
// MINT_FETCH_LDS a thread block carries one more wavefront, the *fetcher*: it
// streams the own rows of the block's wave-channels from HBM, several groups
// ahead, into a ring of LDS per wave-channel, and the wave-channels take them
// from there (LDS operations count on another counter than vector memory).
// Per wave-channel j of the block, in LDS:
//   produced[j]   groups the fetcher has delivered     (fetcher writes)
//   consumed[j]   groups the wave-channel has taken    (wave-channel writes)
//   ring j        fetch_depth x U blocks of 1 KiB, arranged as ll_arrange leaves them
constexpr uint32_t kLdsHeader = 64;       // the two counter arrays (8 wave-channels at most)
struct LdsPort {
    MINT_LDS uint8_t* ring;
    MINT_LDS uint32_t* produced;
    MINT_LDS uint32_t* consumed;
    uint32_t depth;
};
__device__ __forceinline__ uint32_t lds_count(MINT_LDS uint32_t* p) {
    return __builtin_amdgcn_readfirstlane(
        __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP));
}
__device__ __forceinline__ void lds_set(MINT_LDS uint32_t* p, uint32_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ LdsPort lds_port(MINT_LDS uint8_t* base, int j, uint32_t depth, int U) {
    LdsPort port;
    port.produced = reinterpret_cast<MINT_LDS uint32_t*>(base) + j;
    port.consumed = reinterpret_cast<MINT_LDS uint32_t*>(base) + 8 + j;
    port.ring = base + kLdsHeader + (uint32_t)j * depth * (uint32_t)U * kBlockMsg;
    port.depth = depth;
    return port;
}

// The lambdas of the walk are inlined early and kept shallow: every level of
// lambdas capturing lambdas by reference takes the optimiser one more round
// to dissolve, and what it does not dissolve stays in scratch memory (a third
// level left 2.8 KB per lane there and made the copying collectives five
// times slower; the build refuses kernels that use scratch).
#define MINT_INLINE_LAMBDA __attribute__((always_inline))

// The walk of one wave-channel along its rows, specialised by what its
// position does (the flags are compile-time constants so that the loop of an
// origin, an adder, a copier or a sink carries no tests for the other roles).
template <int PROTO, int DT, int CPI, int U, bool LDSF = false, typename RoleT>
__device__ __forceinline__ void ring_walk(const RingArgs& a, const int p, const int h, const int w,
                                          const RoleT role, const LdsPort port = LdsPort{}) {
    constexpr int LDCP = Policy<CPI>::LD, STCP = Policy<CPI>::ST;
    const LaneMap m;
    uint64_t row_bytes;
    uint32_t nblocks, nfull;
    row_extent(a, p, PROTO == PROTO_LL128 ? kBlockRawLL : kBlockRawSimple, row_bytes, nblocks, nfull);
    const uint8_t* in_row = reinterpret_cast<const uint8_t*>(a.input[role.rank]) +
                            (uint64_t)row_read(a, p) * a.row_stride;
    uint8_t* out_row = reinterpret_cast<uint8_t*>(a.output[role.rank]) +
                       (uint64_t)row_written(a, p) * a.row_stride;
    const uint32_t ring_bytes = a.nslots * a.slot_bytes;
    const Window own(reinterpret_cast<const void*>(a.staging[role.rank]), ring_bytes);
    const Window nxt(reinterpret_cast<const void*>(a.staging[role.next]), ring_bytes);
    const uint32_t share_recv = share_of(a, p, h), share_send = share_of(a, p, h + 1);
    const uint32_t own_chan = a.credit_off + (share_recv * (uint32_t)a.waves + (uint32_t)w) * kCreditStride;
    const uint32_t nxt_chan = a.credit_off + (share_send * (uint32_t)a.waves + (uint32_t)w) * kCreditStride;
    uint64_t* own_tail = reinterpret_cast<uint64_t*>(a.staging[role.rank] + own_chan);
    uint64_t* own_head = own_tail + 16;
    uint64_t* nxt_tail = reinterpret_cast<uint64_t*>(a.staging[role.next] + nxt_chan);
    uint64_t* nxt_head = nxt_tail + 16;

    const uint32_t epoch = launch_epoch(a);
    const uint64_t flag_hi = (uint64_t)epoch << 32;        // credit / head words
    const uint32_t W = (uint32_t)a.waves, K = a.k_per_wave;
    const uint32_t groups_per_step = K / U;
    const uint32_t ngroups = a.steps * groups_per_step;
    uint32_t credits_seen = 0, head_seen = 0;
    // wait accounting, 10 ns ticks: only in a library built with
    // -DMINT_RING_STATS (it costs scalar registers, hence occupancy)
#ifdef MINT_RING_STATS
    const bool timing = a.stats != nullptr;
#else
    constexpr bool timing = false;
#endif
    uint64_t t_credit = 0, t_poll = 0, n_repoll = 0, n_groups = 0, t_lds = 0, t_issue = 0;
    const uint64_t t_begin = timing ? wall_clock64() : 0;

    // Group = U blocks of this wave-channel inside one step
    const WalkGeom geom{W, K, a.step_blocks, a.nslots, a.slot_bytes, a.step_msg, nblocks, nfull,
                        (uint32_t)w};
    using Group = mint::Group<U>;
    // load_ll128 of the wave's own rows for one group: only the loads;
    // ll_arrange finishes the job where the values are needed.
    auto load_own = [&](const Group& q, u32x4 (&v)[U]) MINT_INLINE_LAMBDA {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            v[u] = u32x4{0u, 0u, 0u, 0u};
            if (!q.valid[u]) continue;
            if (PROTO == PROTO_LL128) {
                v[u] = ll_fetch_raw(in_row, row_bytes, q.g[u], q.full[u], m);
            } else {
                const uint64_t off = (uint64_t)q.g[u] * kBlockRawSimple + m.lane * 16u;
                v[u] = q.full[u] ? ld128_row(in_row + off)
                                 : load_guarded(in_row, off, 16u, row_bytes);
            }
        }
    };
    // The same for a group that may lie beyond the part of the row made of
    // whole blocks: block numbers are clamped to the last whole block, so the
    // loads are issued unconditionally and always land inside the row (what
    // they bring is only used if the group turns out to be a whole one).
    // Needs nfull >= 1.
    auto fetch_ahead = [&](const Group& q, u32x4 (&v)[U]) MINT_INLINE_LAMBDA {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t g = q.g[u] < nfull ? q.g[u] : nfull - 1u;
            if (PROTO == PROTO_LL128)
                v[u] = ll_fetch_raw(in_row, row_bytes, g, true, m);
            else
                v[u] = ld128_row(in_row + (uint64_t)g * kBlockRawSimple + m.lane * 16u);
        }
    };

    // The own rows of the next whole group, taken out of LDS (LDSF): wait for
    // the fetcher's count, read, hand the ring entry back.  LDS serves a
    // wavefront's operations in order, so the fetcher that sees the new
    // `consumed` knows the reads before it have been done.
    uint32_t lds_taken = 0, lds_entry = 0;
    auto lds_take = [&](u32x4 (&x)[U]) MINT_INLINE_LAMBDA -> bool {
        for (uint32_t spins = 0; lds_count(port.produced) <= lds_taken; ++spins) {
            if (spins >= a.spin_budget || ((spins & 63u) == 63u && aborted(a.status))) return false;
            __builtin_amdgcn_s_sleep(1);
        }
        compiler_fence();
#pragma unroll
        for (int u = 0; u < U; ++u)
            x[u] = *reinterpret_cast<MINT_LDS const u32x4*>(
                port.ring + (lds_entry * (uint32_t)U + (uint32_t)u) * kBlockMsg + m.lane * 16u);
        compiler_fence();
        ++lds_taken;
        lds_entry = lds_entry + 1 == port.depth ? 0 : lds_entry + 1;
        lds_set(port.consumed, lds_taken);
        return true;
    };

    // Own rows of the group being handled and of the one fetched ahead: two
    // register buffers that swap roles from one whole group to the next (the
    // loop over whole groups is unrolled by two).  Copying the fetched-ahead
    // rows into place at the end of a group instead makes every group wait
    // for the fetch it has just issued (a wait for all outstanding loads at
    // the loop's end): a wave-channel's own work per step was 0.80 us that
    // way and is 0.31 us this way.  What that buys depends on the launch
    // geometry - with two slots the wave-channels only arrive earlier at
    // their polls and credit words and re-poll more (0.82 ms against 0.76 for
    // the 8 x 256 MiB reduce-scatter); with three smaller slots they have the
    // slack to use it (0.71 ms), which is the tuned geometry.
    u32x4 rows[2][U];
#pragma unroll
    for (int u = 0; u < U; ++u) rows[0][u] = rows[1][u] = u32x4{0u, 0u, 0u, 0u};
    Group q = Group::first_of(geom);
    uint32_t n = 0;
    // Loop-carried, and looked at in every iteration whether or not a credit
    // was asked for: the compiler then knows that no load into these
    // registers is outstanding at the top of the loop and does not have to
    // drain the memory pipeline (and with it the fetch-ahead) there.
    uint64_t credit_word = 0;

    // One group.  WHOLE = every block of the group lies wholly inside the row:
    // then nothing in the body depends on per-block validity, the own rows of
    // the following group are fetched ahead, and - what the arrangement is
    // for - the number of loads issued after the first polls is the same on
    // every path, so the wait for the polls leaves exactly the fetch-ahead in
    // flight: it has a whole group's time to come back from HBM.  The other
    // groups (the ragged end of a row, a step that is only partly filled) take
    // the guarded body and load their own rows on the spot.
    // Simple protocol, positions that send: the sends of a whole group go out
    // before its saves and before the fetch of the next group's own rows, so
    // that the wait in front of the step counter is a wait for the sends only
    // (adding collectives: reduce-scatter and reduce -1.5 % to -4.5 % against
    // fetching first, where that wait also took in a load from HBM).
    constexpr bool kSendsFirst = PROTO == PROTO_SIMPLE && RoleT::send && !LDSF;
    // Vector-memory operations such a group issues between its sends and the
    // wait in front of the step counter, which may stay in flight there (a
    // wavefront's operations retire in issue order, so waiting until this many
    // are left is waiting for the sends): U saves where the position keeps a
    // copy, U fetches ahead where it has rows of its own - the block under
    // `if (WHOLE && kSendsFirst)` behind the sends - and, for a receiver, the
    // one store of the credit post under `if (q.last)`.  Whoever adds or
    // removes an operation there changes this.
    constexpr int kOpsBehindSends = (RoleT::save ? U : 0) + (RoleT::load ? U : 0) +
                                    (RoleT::recv ? 1 : 0);
    auto run_group = [&](auto whole_tag, auto parity_tag) MINT_INLINE_LAMBDA -> bool {
        constexpr bool WHOLE = decltype(whole_tag)::value;
        constexpr int P = decltype(parity_tag)::value;
        u32x4 (&v)[U] = rows[P];
        u32x4 (&vnext)[U] = rows[P ^ 1];
        const Group qn = q.next(geom);
        const uint32_t s = q.step;
        const uint32_t tag = (epoch << 20) | (s + 1u);
        // wait_ll128 (protocol.py:161-180): the credit for the slot this step
        // goes into is only needed before the send, so its load is issued
        // here, ahead of the polls, and looked at after them.
        const uint32_t need = s >= a.nslots ? s - a.nslots + 1 : 0;
        const bool ask_credit = q.first && role.send && credits_seen < need;
        if (ask_credit) credit_word = ld64_agent(nxt_tail);
        if (q.first && PROTO == PROTO_SIMPLE && role.recv) {
            const uint64_t t0 = timing ? wall_clock64() : 0;
            if (!wait_count(own_head, epoch, s + 1, head_seen, a.spin_budget, a.status)) {
                report_timeout(a.status, p, h, w, s);
                return false;
            }
            if (timing) t_credit += wall_clock64() - t0;
        }
        u32x4 r[U];
        const uint64_t t1 = timing ? wall_clock64() : 0;
        if (role.recv) {
            // first poll of recv_ll128 (protocol.py:102-130): loads only
            compiler_fence();
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (WHOLE || q.valid[u])
                    r[u] = ld128<LDCP>(own, q.msg_off(geom, share_recv, u) + m.lane * 16u);
        }
        if (role.load) {
            if (WHOLE && LDSF) {
                const uint64_t t0 = timing ? wall_clock64() : 0;
                if (!lds_take(v)) {
                    report_timeout(a.status, p, h, w, s);
                    return false;
                }
                if (timing) t_lds += wall_clock64() - t0;
            } else if (WHOLE && kSendsFirst) {
                // (a Simple sender fetches ahead after its sends, see below)
            } else if (WHOLE) {
                fetch_ahead(qn, vnext);
            } else {
                load_own(q, v);
            }
        }
        if (role.recv && PROTO == PROTO_LL128) {
            uint32_t pending = 0;
#pragma unroll
            for (int u = 0; u < U; ++u)
                if ((WHOLE || q.valid[u]) && !wave_all(!m.flag_lane || r[u].w == tag))
                    pending |= 1u << u;
            for (uint32_t spins = 0; pending; ++spins) {
                if (spins >= a.spin_budget || ((spins & 63u) == 63u && aborted(a.status))) {
                    report_timeout(a.status, p, h, w, s);
                    return false;
                }
                __builtin_amdgcn_s_sleep(1);
                compiler_fence();
                ++n_repoll;
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    if (!(pending & (1u << u))) continue;
                    if (ll_poll<LDCP>(own, q.msg_off(geom, share_recv, u), tag, m, r[u]))
                        pending &= ~(1u << u);
                }
            }
        }
        if (timing) { t_poll += wall_clock64() - t1; ++n_groups; }
        if (PROTO == PROTO_LL128 && q.last && role.recv && lane_id() == 0) {
            // post_ll128 (protocol.py:183-189): the tags have been tested, so
            // every line of step s is in registers and the slot is free.  The
            // post goes out ahead of this group's own stores: the sender's
            // credit does not queue behind them.
            if (STCP == CP_NONE) st64_local(own_tail, flag_hi | (uint64_t)(s + 1));
            else st64_agent(own_tail, flag_hi | (uint64_t)(s + 1));
        }
        asm volatile("" : "+v"(credit_word));
        if (ask_credit) {
            const uint64_t t0 = timing ? wall_clock64() : 0;
            const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(credit_word >> 32));
            const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)credit_word);
            if (hi == epoch && lo >= need) {
                credits_seen = lo;
            } else if (!wait_count(nxt_tail, epoch, need, credits_seen, a.spin_budget,
                                   a.status)) {
                report_timeout(a.status, p, h, w, s);
                return false;
            }
            if (timing) t_credit += wall_clock64() - t0;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (!(WHOLE || q.valid[u])) continue;
            const bool full = WHOLE || q.full[u];
            // (rows that came through LDS were arranged by the fetcher)
            u32x4 x = v[u];
            if (role.load && PROTO == PROTO_LL128 && !(WHOLE && LDSF)) x = ll_arrange(x, full, m);
            if (role.recv) {
                if constexpr (DT != DT_BYTES) {
                    x = role.reduce ? ll_comp<DT>(x, r[u]) : r[u];
                } else {
                    x = r[u];
                }
            }
            if (WHOLE && kSendsFirst) {
                // the sends of the whole group first: the counter that follows
                // them then waits for them only
                st128<STCP>(nxt, q.msg_off(geom, share_send, u) + m.lane * 16u, x);
                v[u] = x;
                continue;
            }
            if (role.save) {
                if (PROTO == PROTO_LL128) {
                    ll_save_raw(out_row, row_bytes, q.g[u], full, m, x);
                } else {
                    const uint64_t off = (uint64_t)q.g[u] * kBlockRawSimple + m.lane * 16u;
                    if (full) st128_row(out_row + off, x);
                    else store_guarded(out_row, off, 16u, row_bytes, x);
                }
            }
            if (role.send) {
                if (PROTO == PROTO_LL128)
                    ll_send<STCP>(nxt, q.msg_off(geom, share_send, u), x, tag, m);
                else
                    st128<STCP>(nxt, q.msg_off(geom, share_send, u) + m.lane * 16u, x);
            }
        }
        if (WHOLE && kSendsFirst) {
            compiler_fence();
            if (role.save) {
#pragma unroll
                for (int u = 0; u < U; ++u)
                    st128_row(out_row + (uint64_t)q.g[u] * kBlockRawSimple + m.lane * 16u, v[u]);
            }
            if (role.load) fetch_ahead(qn, vnext);
            compiler_fence();
        }
        if (q.last) {
            // Simple protocol: this wave-channel has taken every line of step s
            // out of its slot (the stores above carry what the loads returned).
            if (PROTO == PROTO_SIMPLE && role.recv && lane_id() == 0) {
                if (STCP == CP_NONE) st64_local(own_tail, flag_hi | (uint64_t)(s + 1));
                else st64_agent(own_tail, flag_hi | (uint64_t)(s + 1));
            }
            if (PROTO == PROTO_SIMPLE && role.send) {
                // Simple protocol: data first, then the step counter.  The data
                // loads of the receiver skip the L1 (LDCP), so no invalidate.
                // Where the group's sends went out first, the operations
                // issued after them - the saves to HBM, the fetch ahead, the
                // credit post - may stay in flight.
                if (WHOLE && kSendsFirst)
                    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kOpsBehindSends) : "memory");
                else
                    wait_stores_visible();
                if (lane_id() == 0) {
                    if (STCP == CP_NONE) st64_local(nxt_head, flag_hi | (uint64_t)(s + 1));
                    else st64_agent(nxt_head, flag_hi | (uint64_t)(s + 1));
                }
            }
        }
        q = qn;
        ++n;
        return true;
    };

    // ---- whole steps, one group per step -----------------------------------
    // s_waitcnt vmcnt retires vector-memory operations in issue order, stores
    // included: a wait for a poll also waits for every store issued before
    // it.  In the loop further down the stores of a step (the sends and, for
    // the copying roles, the saves that go to HBM) are older than the next
    // poll, so each step ends up waiting for their acknowledgement.  When a
    // group is a whole step (k_per_wave == U, the tuned geometries) the order
    // is turned round: the credit word and the first poll of step s + 1 are
    // issued as soon as the tags of step s have been accepted, before step s
    // is added, saved and sent, and the own rows of step s + 2 after that.
    // The stores of a step are then younger than the poll the next step waits
    // for and have a whole step to complete.  Register buffers alternate,
    // hence two copies of the body.  Only the copying collectives run this
    // loop (measured: sendrecv -6 %, broadcast -8 %, allgather -4 %).  A poll
    // issued that early finds its data only if the sender is a full step
    // ahead, which the adding collectives - every position waiting for its
    // own rows from HBM - are not: their early polls fail and are repeated,
    // and reducescatter lost 12 %.
    //
    // The compiler derives every wait from the number of memory operations
    // issued after the one it needs and takes the smaller number where paths
    // meet.  So nothing in the body is issued conditionally (the tail post is
    // stored by all lanes, fetch addresses are clamped), a wave that gives up
    // ends on the spot instead of leaving the loop, and the prologue issues
    // exactly the queue a later step finds (stand-ins for the stores go to an
    // unused part of a credit line of this wave-channel: the one it looks at
    // when it sends, else its own).
    //
    // An origin of a copying collective (it loads rows and sends them, and
    // receives nothing) has its own loop under the XCD-local policy.  Its
    // only vector loads are the row fetches; the one word it has to look at,
    // the credit, it reads through the scalar unit, which counts apart.  So
    // the fetches run kOriginDepth steps ahead and a wait for the oldest
    // leaves the younger ones in flight: a load from HBM takes 2.5 us under a
    // collective's stores, twice a step.
    constexpr int kOriginDepth = 4;
    constexpr bool kDeepOrigin = PROTO == PROTO_LL128 && DT == DT_BYTES && STCP == CP_NONE &&
                                 RoleT::load && RoleT::send && !RoleT::recv && !RoleT::save &&
                                 U <= 2;
    // (Only where CUs are set apart for the origins: an origin that shares
    // its CU's memory pipeline gains nothing from more loads in flight -
    // sendrecv and alltoall take 3 - 7 % longer with this loop.)
    bool origin_done = false;
    if constexpr (kDeepOrigin) {
      if (a.origin_cus && K == (uint32_t)U && ngroups) {
        origin_done = true;
        const uint32_t last_idx = (uint32_t)(U - 1) * W + (uint32_t)w;
        uint32_t whole_steps = nfull > last_idx ? (nfull - 1u - last_idx) / a.step_blocks + 1u : 0u;
        if (whole_steps > a.steps) whole_steps = a.steps;
        if (whole_steps) {
            u32x4 vv[kOriginDepth][U];
            uint32_t step = 0, slot = 0;
            auto fetch_step = [&](uint32_t of_step, u32x4 (&x)[U]) MINT_INLINE_LAMBDA {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    uint32_t g = of_step * a.step_blocks + (uint32_t)u * W + (uint32_t)w;
                    g = g < nfull ? g : nfull - 1u;      // beyond the whole blocks: any valid address
                    x[u] = ll_fetch_raw(in_row, row_bytes, g, true, m);
                }
            };
            // The queue a later step finds when it waits for its rows: per step
            // fetched ahead, U sends and the fetch.  The prologue issues the same
            // (the compiler takes the smaller count where paths meet); stand-ins
            // for the sends go to an unused part of the credit line this
            // wave-channel looks at.
            uint64_t* const pad = nxt_tail + 8;
            fetch_step(0u, vv[0]);
#pragma unroll
            for (int d = 1; d < kOriginDepth; ++d) {
                compiler_fence();
#pragma unroll
                for (int u = 0; u < U; ++u) st64_local(pad, 0ull);
                compiler_fence();
                fetch_step((uint32_t)d, vv[d]);
            }
            auto origin_step = [&](auto phase) MINT_INLINE_LAMBDA {
                constexpr int B = decltype(phase)::value;
                const uint32_t tag = (epoch << 20) | (step + 1u);
                const uint32_t need = step >= a.nslots ? step - a.nslots + 1 : 0;
                const uint32_t send_base = slot * a.slot_bytes + share_send * a.step_msg;
                // wait_ll128 (protocol.py:161-180)
                const uint64_t t0 = timing ? wall_clock64() : 0;
                for (uint32_t spins = 0; credits_seen < need; ++spins) {
                    const uint64_t cw = ld64_scalar(nxt_tail);
                    if ((uint32_t)(cw >> 32) == epoch && (uint32_t)cw >= need) {
                        credits_seen = (uint32_t)cw;
                        break;
                    }
                    if (spins >= a.spin_budget ||
                        ((spins & 63u) == 63u &&
                         __builtin_amdgcn_readfirstlane(ld32_agent_apart(a.status + 3)) != 0u)) {
                        report_timeout(a.status, p, h, w, step);
                        __builtin_amdgcn_endpgm();
                    }
                    __builtin_amdgcn_s_sleep(1);
                }
                if (timing) {
                    const uint64_t t1 = wall_clock64();
                    t_credit += t1 - t0;
#pragma unroll
                    for (int u = 0; u < U; ++u) asm volatile("" : "+v"(vv[B][u]));
                    t_lds += wall_clock64() - t1;
                }
                ++n_groups;
                const uint64_t t2 = timing ? wall_clock64() : 0;
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const uint32_t idx = (uint32_t)u * W + (uint32_t)w;
                    ll_send<STCP>(nxt, send_base + idx * kBlockMsg, ll_arrange(vv[B][u], true, m), tag, m);
                }
                compiler_fence();
                fetch_step(step + (uint32_t)kOriginDepth, vv[B]);
                if (timing) {
                    compiler_fence();
                    t_issue += wall_clock64() - t2;
                }
                slot = slot + 1 == a.nslots ? 0 : slot + 1;
                ++step;
            };
            static_assert(kOriginDepth == 4, "the loop below is unrolled by the depth");
            while (step < whole_steps) {
                origin_step(std::integral_constant<int, 0>{});
                if (step >= whole_steps) break;
                origin_step(std::integral_constant<int, 1>{});
                if (step >= whole_steps) break;
                origin_step(std::integral_constant<int, 2>{});
                if (step >= whole_steps) break;
                origin_step(std::integral_constant<int, 3>{});
            }
            q.step = step; q.slot = slot; q.k0 = 0;
            q.fill(geom);
            n = step;
        }
      }
    }
    // ---- whole steps of the adding collectives ---------------------------------
    // The same step as run_group's - credit word, polls, fetch of the next
    // step's own rows, tags, credit post, add, save / send - with everything
    // that does not change from step to step taken out of it: a CU has one
    // scalar unit for its sixteen wavefronts, and the general group above
    // spends 76 scalar instructions and 9 branches per step on bookkeeping
    // (which group of the step, which blocks are valid, what the next group
    // looks like).  The polls' staging offsets ride in the scalar offset of the
    // buffer instruction, the row pointer and the tag advance by constants.
    // Nothing is issued conditionally except the credit load (fetch addresses
    // are clamped into the row), so every wait leaves exactly the fetch ahead
    // in flight.  Steps that are not whole take the general path.
    if constexpr (PROTO == PROTO_LL128 && DT != DT_BYTES && !LDSF) {
      if (K == (uint32_t)U && ngroups) {
        const uint32_t last_idx = (uint32_t)(U - 1) * W + (uint32_t)w;
        uint32_t whole_steps = nfull > last_idx ? (nfull - 1u - last_idx) / a.step_blocks + 1u : 0u;
        if (whole_steps > a.steps) whole_steps = a.steps;
        if (whole_steps) {
            u32x4 vv[2][U];
            // What moves from step to step: the tag, the credits the step needs
            // (positive from step nslots on), the first block, the slot's offset.
            uint32_t slot_off = 0;
            uint32_t tag = (epoch << 20) | 1u;
            const uint32_t end_tag = tag + whole_steps;
            int32_t need = 1 - (int32_t)a.nslots;
            const uint32_t recv_v = share_recv * a.step_msg + (uint32_t)w * kBlockMsg + m.lane * 16u;
            const uint32_t send_v = share_send * a.step_msg + (uint32_t)w * kBlockMsg + m.lane * 16u;
            const uint32_t last_full = nfull - 1u;
            constexpr uint64_t kDataLanes = 0x7777777777777777ull;    // every lane but the fourth of a sector
            uint32_t g0 = (uint32_t)w;                      // block u = 0 of the step in hand
            uint64_t cw = 0;
            auto fetch_step = [&](uint32_t first, u32x4 (&x)[U]) MINT_INLINE_LAMBDA {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    uint32_t g = first + (uint32_t)u * W;
                    g = g < last_full ? g : last_full;       // beyond the whole blocks: any valid address
                    x[u] = ll_fetch_raw(in_row, row_bytes, g, true, m);
                }
            };
            auto give_up = [&]() MINT_INLINE_LAMBDA {
                report_timeout(a.status, p, h, w, (uint32_t)(need + (int32_t)a.nslots) - 1u);
                __builtin_amdgcn_endpgm();
            };
            auto lean_step = [&](auto phase) MINT_INLINE_LAMBDA {
                constexpr int B = decltype(phase)::value, B1 = B ^ 1;
                u32x4 r[U];
                // wait_ll128 (protocol.py:161-180): asked for ahead of the polls, looked at after them
                if (role.send && (int32_t)credits_seen < need) cw = ld64_agent(nxt_tail);
                const uint64_t t1 = timing ? wall_clock64() : 0;
                if (role.recv) {
                    compiler_fence();
#pragma unroll
                    for (int u = 0; u < U; ++u)
                        r[u] = ld128<LDCP>(own, recv_v + (uint32_t)u * W * kBlockMsg, slot_off);
                }
                compiler_fence();
                if (role.load) fetch_step(g0 + a.step_blocks, vv[B1]);
                compiler_fence();
                if (role.recv) {
                    // recv_ll128 (protocol.py:102-130)
                    uint32_t pending = 0;
#pragma unroll
                    for (int u = 0; u < U; ++u)
                        if ((__ballot(r[u].w == tag) | kDataLanes) != ~0ull) pending |= 1u << u;
                    for (uint32_t spins = 0; pending; ++spins) {
                        if (spins >= a.spin_budget || ((spins & 63u) == 63u && aborted(a.status)))
                            give_up();
                        __builtin_amdgcn_s_sleep(1);
                        compiler_fence();
                        ++n_repoll;
#pragma unroll
                        for (int u = 0; u < U; ++u) {
                            if (!(pending & (1u << u))) continue;
                            r[u] = ld128<LDCP>(own, recv_v + (uint32_t)u * W * kBlockMsg, slot_off);
                            if ((__ballot(r[u].w == tag) | kDataLanes) == ~0ull)
                                pending &= ~(1u << u);
                        }
                    }
                    // post_ll128 (protocol.py:183-189): the step is in registers,
                    // the slot is free; every lane stores the same word
                    // From here to the step's stores the wavefront has what it needs:
                    // it goes ahead of the wavefronts of its SIMD that would only
                    // issue another poll (-0.5 % on the 8 x 256 MiB reduce-scatter).
                    __builtin_amdgcn_s_setprio(3);
                    const uint64_t posted = flag_hi | (uint64_t)(uint32_t)(need + (int32_t)a.nslots);
                    if (STCP == CP_NONE) st64_local(own_tail, posted);
                    else st64_agent(own_tail, posted);
                }
                if (timing) { t_poll += wall_clock64() - t1; ++n_groups; }
                asm volatile("" : "+v"(cw));
                if (role.send && (int32_t)credits_seen < need) {
                    const uint64_t t0 = timing ? wall_clock64() : 0;
                    // (compared in vector registers: every lane holds the word)
                    if (__ballot((uint32_t)(cw >> 32) == epoch && (int32_t)(uint32_t)cw >= need) != 0ull)
                        credits_seen = __builtin_amdgcn_readfirstlane((uint32_t)cw);
                    else if (!wait_count(nxt_tail, epoch, (uint32_t)need, credits_seen, a.spin_budget,
                                         a.status))
                        give_up();
                    if (timing) t_credit += wall_clock64() - t0;
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    u32x4 x = vv[B][u];
                    if (role.load) x = ll_arrange(x, true, m);
                    if (role.recv) x = role.reduce ? ll_comp<DT>(x, r[u]) : r[u];
                    if (role.save) ll_save_raw(out_row, row_bytes, g0 + (uint32_t)u * W, true, m, x);
                    if (role.send) {
                        if (m.flag_lane) x.w = tag;
                        st128<STCP>(nxt, send_v + (uint32_t)u * W * kBlockMsg + slot_off, x);
                    }
                }
                if (role.recv) __builtin_amdgcn_s_setprio(0);
                ++tag; ++need;
                g0 += a.step_blocks;
                slot_off += a.slot_bytes;
                slot_off = slot_off == ring_bytes ? 0u : slot_off;
            };
            // an odd number of steps starts with one step out of the second
            // buffer, so that the loop is whole pairs and has one way out
            if (whole_steps & 1u) {
                if (role.load) fetch_step(g0, vv[1]);
                lean_step(std::integral_constant<int, 1>{});
            } else if (role.load) {
                fetch_step(g0, vv[0]);
            }
            while (tag != end_tag) {
                lean_step(std::integral_constant<int, 0>{});
                lean_step(std::integral_constant<int, 1>{});
            }
            const uint32_t step = whole_steps, slot = slot_off / a.slot_bytes;
            // what is left (a ragged or partly filled last step) starts afresh
            q.step = step; q.slot = slot; q.k0 = 0;
            q.fill(geom);
            n = step;
        }
      }
    }
    // ---- whole steps of the Simple protocol ------------------------------------
    // The whole group of run_group for the Simple protocol (step counter,
    // data loads, credit, sends first, saves, fetch ahead, credit post, wait
    // for the sends, step counter for the next rank) without the bookkeeping,
    // as above: the general group spends 16 scalar instructions per
    // vector-memory instruction.  All element types and roles.
    if constexpr (PROTO == PROTO_SIMPLE && !LDSF) {
      if (K == (uint32_t)U && ngroups) {
        const uint32_t last_idx = (uint32_t)(U - 1) * W + (uint32_t)w;
        uint32_t whole_steps = nfull > last_idx ? (nfull - 1u - last_idx) / a.step_blocks + 1u : 0u;
        if (whole_steps > a.steps) whole_steps = a.steps;
        if (whole_steps) {
            u32x4 vv[2][U];
            uint32_t slot_off = 0;
            uint32_t count = 1;                              // steps done with this one
            const uint32_t end_count = 1u + whole_steps;
            int32_t need = 1 - (int32_t)a.nslots;
            const uint32_t recv_v = share_recv * a.step_msg + (uint32_t)w * kBlockMsg + m.lane * 16u;
            const uint32_t send_v = share_send * a.step_msg + (uint32_t)w * kBlockMsg + m.lane * 16u;
            const uint32_t last_full = nfull - 1u;
            uint32_t g0 = (uint32_t)w;
            uint64_t cw = 0;
            // Operations between a step's sends and the wait in front of its
            // step counter (see kOpsBehindSends): saves, fetch ahead, credit post.
            constexpr int kBehind = (RoleT::save ? U : 0) + (RoleT::load ? U : 0) + (RoleT::recv ? 1 : 0);
            auto fetch_step = [&](uint32_t first, u32x4 (&x)[U]) MINT_INLINE_LAMBDA {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    uint32_t g = first + (uint32_t)u * W;
                    g = g < last_full ? g : last_full;       // beyond the whole blocks: any valid address
                    x[u] = ld128_row(in_row + (uint64_t)g * kBlockRawSimple + m.lane * 16u);
                }
            };
            auto give_up = [&]() MINT_INLINE_LAMBDA {
                report_timeout(a.status, p, h, w, count - 1u);
                __builtin_amdgcn_endpgm();
            };
            auto lean_step = [&](auto phase) MINT_INLINE_LAMBDA {
                constexpr int B = decltype(phase)::value, B1 = B ^ 1;
                u32x4 r[U];
                if (role.send && (int32_t)credits_seen < need) cw = ld64_agent(nxt_tail);
                if (role.recv) {
                    // the sender's step counter: every line of this step is in the slot
                    // (its wait is booked with the credits)
                    const uint64_t t0 = timing ? wall_clock64() : 0;
                    if (head_seen < count) {
                        const uint64_t hw = ld64_agent(own_head);
                        if (__ballot((uint32_t)(hw >> 32) == epoch && (uint32_t)hw >= count) != 0ull)
                            head_seen = __builtin_amdgcn_readfirstlane((uint32_t)hw);
                        else if (!wait_count(own_head, epoch, count, head_seen, a.spin_budget, a.status))
                            give_up();
                    }
                    if (timing) t_credit += wall_clock64() - t0;
                    compiler_fence();
#pragma unroll
                    for (int u = 0; u < U; ++u)
                        r[u] = ld128<LDCP>(own, recv_v + (uint32_t)u * W * kBlockMsg, slot_off);
                    compiler_fence();
                }
                if (timing) ++n_groups;
                asm volatile("" : "+v"(cw));
                if (role.send && (int32_t)credits_seen < need) {
                    const uint64_t t0 = timing ? wall_clock64() : 0;
                    if (__ballot((uint32_t)(cw >> 32) == epoch && (int32_t)(uint32_t)cw >= need) != 0ull)
                        credits_seen = __builtin_amdgcn_readfirstlane((uint32_t)cw);
                    else if (!wait_count(nxt_tail, epoch, (uint32_t)need, credits_seen, a.spin_budget,
                                         a.status))
                        give_up();
                    if (timing) t_credit += wall_clock64() - t0;
                }
                u32x4 x[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    x[u] = vv[B][u];
                    if (role.recv) {
                        if constexpr (DT != DT_BYTES) {
                            x[u] = role.reduce ? ll_comp<DT>(x[u], r[u]) : r[u];
                        } else {
                            x[u] = r[u];
                        }
                    }
                    if (role.send) st128<STCP>(nxt, send_v + (uint32_t)u * W * kBlockMsg + slot_off, x[u]);
                }
                compiler_fence();
                if (role.save) {
#pragma unroll
                    for (int u = 0; u < U; ++u)
                        st128_row(out_row + (uint64_t)(g0 + (uint32_t)u * W) * kBlockRawSimple + m.lane * 16u, x[u]);
                }
                if (role.load) fetch_step(g0 + a.step_blocks, vv[B1]);
                compiler_fence();
                if (role.recv) {
                    // every line of the step has been taken out of the slot (the
                    // stores above carry what the loads returned)
                    const uint64_t posted = flag_hi | (uint64_t)count;
                    if (STCP == CP_NONE) st64_local(own_tail, posted);
                    else st64_agent(own_tail, posted);
                }
                if (role.send) {
                    // data first, then the step counter; what was issued behind
                    // the sends may stay in flight
                    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kBehind) : "memory");
                    const uint64_t posted = flag_hi | (uint64_t)count;
                    if (STCP == CP_NONE) st64_local(nxt_head, posted);
                    else st64_agent(nxt_head, posted);
                }
                ++count; ++need;
                g0 += a.step_blocks;
                slot_off += a.slot_bytes;
                slot_off = slot_off == ring_bytes ? 0u : slot_off;
            };
            if (whole_steps & 1u) {
                if (role.load) fetch_step(g0, vv[1]);
                lean_step(std::integral_constant<int, 1>{});
            } else if (role.load) {
                fetch_step(g0, vv[0]);
            }
            while (count != end_count) {
                lean_step(std::integral_constant<int, 0>{});
                lean_step(std::integral_constant<int, 1>{});
            }
            const uint32_t step = whole_steps, slot = slot_off / a.slot_bytes;
            q.step = step; q.slot = slot; q.k0 = 0;
            q.fill(geom);
            n = step;
        }
      }
    }
    if constexpr (PROTO == PROTO_LL128 && DT == DT_BYTES) {
      if (!origin_done && K == (uint32_t)U && ngroups) {
        const uint32_t last_idx = (uint32_t)(U - 1) * W + (uint32_t)w;
        uint32_t whole_steps = nfull > last_idx ? (nfull - 1u - last_idx) / a.step_blocks + 1u : 0u;
        if (whole_steps > a.steps) whole_steps = a.steps;
        if (whole_steps) {
            u32x4 rr[2][U], vv[2][U];
            uint64_t cw[2] = {0, 0};
            uint32_t step = 0, slot = 0;
            auto poll_step = [&](uint32_t at_slot, u32x4 (&r)[U]) MINT_INLINE_LAMBDA {
                const uint32_t base = at_slot * a.slot_bytes + share_recv * a.step_msg;
#pragma unroll
                for (int u = 0; u < U; ++u)
                    r[u] = ld128<LDCP>(own, base + ((uint32_t)u * W + (uint32_t)w) * kBlockMsg +
                                                m.lane * 16u);
            };
            auto fetch_step = [&](uint32_t of_step, u32x4 (&x)[U]) MINT_INLINE_LAMBDA {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    uint32_t g = of_step * a.step_blocks + (uint32_t)u * W + (uint32_t)w;
                    g = g < nfull ? g : nfull - 1u;      // beyond the whole blocks: any valid address
                    x[u] = ll_fetch_raw(in_row, row_bytes, g, true, m);
                }
            };
            // (an origin need not have staging of its own)
            uint64_t* const pad = role.send ? nxt_tail + 8 : own_tail + 8;
            auto store_pad = [&]() MINT_INLINE_LAMBDA {
                if (STCP == CP_NONE) st64_local(pad, 0ull);
                else st64_agent(pad, 0ull);
            };
            auto give_up = [&]() MINT_INLINE_LAMBDA {
                report_timeout(a.status, p, h, w, step);
                __builtin_amdgcn_endpgm();
            };
            if (role.load) fetch_step(0, vv[0]);
            compiler_fence();
            if (role.send) cw[0] = ld64_agent(nxt_tail);
            if (role.recv) poll_step(0, rr[0]);
            compiler_fence();
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (role.save) store_pad();
                if (role.send) store_pad();
            }
            compiler_fence();
            if (role.load) fetch_step(1, vv[1]);
            auto whole_step = [&](auto phase) MINT_INLINE_LAMBDA {
                constexpr int B = decltype(phase)::value, B1 = B ^ 1;
                const uint32_t next_slot = slot + 1 == a.nslots ? 0 : slot + 1;
                const uint32_t tag = (epoch << 20) | (step + 1u);
                const uint32_t need = step >= a.nslots ? step - a.nslots + 1 : 0;
                const uint32_t recv_base = slot * a.slot_bytes + share_recv * a.step_msg;
                const uint32_t send_base = slot * a.slot_bytes + share_send * a.step_msg;
                const uint64_t t1 = timing ? wall_clock64() : 0;
                if (role.recv) {
                    uint32_t pending = 0;
#pragma unroll
                    for (int u = 0; u < U; ++u)
                        if (!wave_all(!m.flag_lane || rr[B][u].w == tag)) pending |= 1u << u;
                    for (uint32_t spins = 0; pending; ++spins) {
                        if (spins >= a.spin_budget || ((spins & 63u) == 63u && aborted(a.status)))
                            give_up();
                        __builtin_amdgcn_s_sleep(1);
                        compiler_fence();
                        ++n_repoll;
#pragma unroll
                        for (int u = 0; u < U; ++u) {
                            if (!(pending & (1u << u))) continue;
                            if (ll_poll<LDCP>(own, recv_base + ((uint32_t)u * W + (uint32_t)w) * kBlockMsg,
                                              tag, m, rr[B][u]))
                                pending &= ~(1u << u);
                        }
                    }
                }
                ++n_groups;
                if (timing) t_poll += wall_clock64() - t1;
                if (role.recv) {
                    // post_ll128 (protocol.py:183-189), as soon as the step is in
                    // registers and ahead of this step's own stores, so that the
                    // credit does not queue behind them; every lane stores the
                    // same word
                    if (STCP == CP_NONE) st64_local(own_tail, flag_hi | (uint64_t)(step + 1));
                    else st64_agent(own_tail, flag_hi | (uint64_t)(step + 1));
                }
                if (timing && role.load) {
                    // how long the own rows fetched two steps ago still take to arrive
                    const uint64_t t0 = wall_clock64();
#pragma unroll
                    for (int u = 0; u < U; ++u) asm volatile("" : "+v"(vv[B][u]));
                    t_lds += wall_clock64() - t0;
                }
                if (role.send) {
                    const uint64_t t0 = timing ? wall_clock64() : 0;
                    asm volatile("" : "+v"(cw[B]));
                    if (credits_seen < need) {
                        const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(cw[B] >> 32));
                        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)cw[B]);
                        if (hi == epoch && lo >= need) credits_seen = lo;
                        else if (!wait_count(nxt_tail, epoch, need, credits_seen, a.spin_budget,
                                             a.status))
                            give_up();
                    }
                    if (timing) t_credit += wall_clock64() - t0;
                }
                // the next step's credit word and first poll go out ahead of this step's stores
                compiler_fence();
                const uint64_t t2 = timing ? wall_clock64() : 0;
                if (role.send) cw[B1] = ld64_agent(nxt_tail);
                if (role.recv) poll_step(next_slot, rr[B1]);
                compiler_fence();
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const uint32_t idx = (uint32_t)u * W + (uint32_t)w;
                    u32x4 x = vv[B][u];
                    if (role.load) x = ll_arrange(x, true, m);
                    if (role.recv) {
                        if constexpr (DT != DT_BYTES) {
                            x = role.reduce ? ll_comp<DT>(x, rr[B][u]) : rr[B][u];
                        } else {
                            x = rr[B][u];
                        }
                    }
                    if (role.save)
                        ll_save_raw(out_row, row_bytes, step * a.step_blocks + idx, true, m, x);
                    if (role.send) ll_send<STCP>(nxt, send_base + idx * kBlockMsg, x, tag, m);
                }
                compiler_fence();
                if (role.load) fetch_step(step + 2u, vv[B]);
                if (timing) {
                    // how long the step's loads and stores took to issue
                    compiler_fence();
                    t_issue += wall_clock64() - t2;
                }
                slot = next_slot;
                ++step;
            };
            while (step < whole_steps) {
                whole_step(std::integral_constant<int, 0>{});
                if (step >= whole_steps) break;
                whole_step(std::integral_constant<int, 1>{});
            }
            // what is left (a ragged or partly filled last step) starts afresh
            q.step = step; q.slot = slot; q.k0 = 0;
            q.fill(geom);
            n = step;
        }
      }
    }

    // block numbers grow from group to group, so the whole groups come first
    using Even = std::integral_constant<int, 0>;
    using Odd = std::integral_constant<int, 1>;
    if (!LDSF && role.load && n < ngroups && q.g[U - 1] < nfull) fetch_ahead(q, rows[0]);
    while (n < ngroups && q.g[U - 1] < nfull) {
        if (!run_group(std::true_type{}, Even{})) return;
        if (!(n < ngroups && q.g[U - 1] < nfull)) break;
        if (!run_group(std::true_type{}, Odd{})) return;
    }
    while (n < ngroups)
        if (!run_group(std::false_type{}, Even{})) return;

    if (timing && lane_id() == 0) {
        unsigned long long* st = reinterpret_cast<unsigned long long*>(a.stats) + 8 * h;
        atomicAdd(st + 0, (unsigned long long)n_groups);
        atomicAdd(st + 1, (unsigned long long)n_repoll);
        atomicAdd(st + 2, (unsigned long long)t_credit);
        atomicAdd(st + 3, (unsigned long long)t_poll);
        atomicAdd(st + 4, (unsigned long long)(wall_clock64() - t_begin));
        atomicAdd(st + 5, 1ull);
        atomicAdd(st + 6, (unsigned long long)t_lds);
        atomicAdd(st + 7, (unsigned long long)t_issue);
    }
}

// One specialised walk per role.
template <int PROTO, int DT, int CPI, int U, bool LDSF>
__device__ __forceinline__ void walk_as(const RingArgs& a, const int p, const int h, const int w,
                                        const Role role, const LdsPort port = LdsPort{}) {
    const int rk = role.rank, nx = role.next;
    if (!role.recv) {
        ring_walk<PROTO, DT, CPI, U, LDSF>(a, p, h, w, FixedRole<true, false, false, false, true>{rk, nx}, port);
    } else if (role.reduce) {
        if constexpr (DT != DT_BYTES) {
            if (role.save)
                ring_walk<PROTO, DT, CPI, U, LDSF>(a, p, h, w, FixedRole<true, true, true, true, true>{rk, nx}, port);
            else
                ring_walk<PROTO, DT, CPI, U, LDSF>(a, p, h, w, FixedRole<true, true, true, false, true>{rk, nx}, port);
        }
    } else if (role.send) {
        if (role.save)
            ring_walk<PROTO, DT, CPI, U>(a, p, h, w, FixedRole<false, true, false, true, true>{rk, nx});
        else
            ring_walk<PROTO, DT, CPI, U>(a, p, h, w, FixedRole<false, true, false, false, true>{rk, nx});
    } else {
        ring_walk<PROTO, DT, CPI, U>(a, p, h, w, FixedRole<false, true, false, true, false>{rk, nx});
    }
}

template <int PROTO, int DT, int CPI, int U>
__global__ void __launch_bounds__(512) ring_kernel(const RingArgs a) {
    // the wave index is the same in every lane: keep it (and all the index
    // arithmetic that hangs off it) in scalar registers
    __shared__ int entry[1];
    const int wpb = (int)(blockDim.x >> 6);
    const int wib = (int)__builtin_amdgcn_readfirstlane((uint32_t)wave_in_block());
    const Seat st = take_seat(a, wpb, wib, wib, (MINT_LDS int*)entry);
    if (!st.ok) return;
    // (plain integers from here on: a seat handed on by reference stays in
    // scratch memory)
    const int p = st.p, h = st.h, w = st.w;
    const Role role = role_of(a, p, h);
    walk_as<PROTO, DT, CPI, U, false>(a, p, h, w, role);
}

// The fetcher wavefront of a thread block (MINT_FETCH_LDS): streams the own
// rows of the block's WPB wave-channels into their LDS rings, R groups of
// every wave-channel in flight in registers.  Wave-channel j of the block
// handles, in group n, the blocks  step * step_blocks + (k0 + u) * W + w0 + j
// (the walk of Group<U>); only whole groups come through LDS, the ragged end
// of a row is loaded by the wave-channel itself.  Loads are issued
// unconditionally (block numbers clamped into the row) so that the number of
// loads in flight behind the one being delivered is the same on every path.
template <int U, int WPB, int R>
__device__ __forceinline__ void row_fetcher(const RingArgs& a, const Seat& st, const Role& role,
                                            MINT_LDS uint8_t* lds) {
    const LaneMap m;
    uint64_t row_bytes;
    uint32_t nblocks, nfull;
    row_extent(a, st.p, kBlockRawLL, row_bytes, nblocks, nfull);
    if (nfull == 0) return;
    const uint8_t* in_row = reinterpret_cast<const uint8_t*>(a.input[role.rank]) +
                            (uint64_t)st.p * a.row_stride;
    const uint32_t W = (uint32_t)a.waves, K = a.k_per_wave, depth = a.fetch_depth;
    const uint32_t ngroups = a.steps * (K / (uint32_t)U);
    const uint32_t w0 = (uint32_t)seat_wave(a, st.gw, WPB, 0);
    const int left = a.waves - st.gw * WPB;
    const int nworkers = left < WPB ? left : WPB;
    struct Cursor {
        uint32_t step, k0;
        __device__ __forceinline__ void advance(uint32_t K) {
            k0 += (uint32_t)U;
            if (k0 >= K) { k0 = 0; ++step; }
        }
    };
    auto block_of = [&](const Cursor& c, int j, int u) {
        return c.step * a.step_blocks + (c.k0 + (uint32_t)u) * W + w0 + (uint32_t)j;
    };
    u32x4 x[R][WPB][U];
    Cursor ci{0u, 0u};
    auto issue = [&](int r) {
#pragma unroll
        for (int j = 0; j < WPB; ++j)
#pragma unroll
            for (int u = 0; u < U; ++u) {
                uint32_t g = block_of(ci, j, u);
                g = g < nfull ? g : nfull - 1u;
                x[r][j][u] = ll_fetch_raw(in_row, row_bytes, g, true, m);
            }
        ci.advance(K);
    };
#pragma unroll
    for (int r = 0; r < R; ++r) issue(r);
    Cursor cd{0u, 0u};
    uint32_t n = 0, entry = 0;
    uint32_t freed[WPB];
#pragma unroll
    for (int j = 0; j < WPB; ++j) freed[j] = 0;
#ifdef MINT_RING_STATS
    const bool timing = a.stats != nullptr;
#else
    constexpr bool timing = false;
#endif
    uint64_t t_room = 0;
    auto leave = [&]() {
        if (timing && lane_id() == 0)
            atomicAdd(reinterpret_cast<unsigned long long*>(a.stats) + 8 * st.h + 7,
                      (unsigned long long)t_room);
    };
    for (;;) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            // block numbers grow with j: when wave-channel 0 has no whole group left, nobody has
            if (n >= ngroups || block_of(cd, 0, U - 1) >= nfull) { leave(); return; }
            const uint64_t t0 = timing ? wall_clock64() : 0;
#pragma unroll
            for (int j = 0; j < WPB; ++j) {
                if (j >= nworkers || block_of(cd, j, U - 1) >= nfull) continue;
                const LdsPort port = lds_port(lds, j, depth, U);
                // room in the ring: the wave-channel has taken group n - depth
                for (uint32_t spins = 0; n >= freed[j] + depth; ++spins) {
                    freed[j] = lds_count(port.consumed);
                    if (n < freed[j] + depth) break;
                    if (spins >= a.spin_budget || ((spins & 63u) == 63u && aborted(a.status))) {
                        report_timeout(a.status, st.p, st.h, (int)(w0 + (uint32_t)j), n);
                        return;
                    }
                    __builtin_amdgcn_s_sleep(1);
                }
                if (timing && j == WPB - 1) t_room += wall_clock64() - t0;
#pragma unroll
                for (int u = 0; u < U; ++u)
                    *reinterpret_cast<MINT_LDS u32x4*>(
                        port.ring + (entry * (uint32_t)U + (uint32_t)u) * kBlockMsg + m.lane * 16u) =
                        ll_arrange(x[r][j][u], true, m);
            }
            // LDS serves this wavefront's operations in order: the counts go
            // out behind the data
            compiler_fence();
#pragma unroll
            for (int j = 0; j < WPB; ++j)
                if (j < nworkers && block_of(cd, j, U - 1) < nfull)
                    lds_set(lds_port(lds, j, depth, U).produced, n + 1u);
            compiler_fence();
            issue(r);
            cd.advance(K);
            ++n;
            entry = entry + 1 == depth ? 0 : entry + 1;
        }
    }
}

// The ring kernel with own rows through LDS: WPB wave-channels and one fetcher
// per thread block.  LL128, reducing ops.
template <int DT, int CPI, int U, int WPB, int R>
__global__ void __launch_bounds__((WPB + 1) * 64) ring_kernel_lds(const RingArgs a) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    MINT_LDS uint8_t* lds = (MINT_LDS uint8_t*)lds_raw;
    __shared__ int entry[1];
    if (threadIdx.x < 16) reinterpret_cast<MINT_LDS uint32_t*>(lds)[threadIdx.x] = 0u;
    __syncthreads();
    const int wib = (int)__builtin_amdgcn_readfirstlane((uint32_t)wave_in_block());
    const bool fetcher = wib == WPB;
    const Seat st = take_seat(a, WPB, fetcher ? 0 : wib, wib, (MINT_LDS int*)entry);
    if (!st.ok) return;
    const Role role = role_of(a, st.p, st.h);
    if (fetcher) {
        if (role.load) row_fetcher<U, WPB, R>(a, st, role, lds);
        return;
    }
    walk_as<PROTO_LL128, DT, CPI, U, true>(a, st.p, st.h, st.w, role,
                                           lds_port(lds, wib, a.fetch_depth, U));
}

}  // namespace mint
