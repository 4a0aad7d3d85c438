// Stand-alone kernels: simple-protocol copy, LL128 codec, element sum,
// torn-line probe, block -> XCD map.
#pragma once
#include "protocol.hpp"

namespace mint {

// recv_kernel (1_sendrecv_direct.py:31-54): persistent copy, 16 bytes per
// lane, four independent accesses in flight per lane.  Every block walks a
// contiguous share of the buffer (measured: a grid-stride walk loses up to a
// fifth of the HBM bandwidth once the grid exceeds one block per CU).
__global__ void __launch_bounds__(1024) copy_simple_kernel(const uint8_t* __restrict__ src,
                                                           uint8_t* __restrict__ dst,
                                                           uint64_t nbytes) {
    const uint64_t nvec = nbytes >> 4;
    const uint64_t per = (nvec + gridDim.x - 1) / gridDim.x;
    const uint64_t lo = (uint64_t)blockIdx.x * per;
    const uint64_t hi = lo + per < nvec ? lo + per : nvec;
    const uint64_t nthr = blockDim.x;
    uint64_t i = lo + threadIdx.x;
    for (; i + 3 * nthr < hi; i += 4 * nthr) {
        u32x4 a = ld128_stream(src + (i << 4));
        u32x4 b = ld128_stream(src + ((i + nthr) << 4));
        u32x4 c = ld128_stream(src + ((i + 2 * nthr) << 4));
        u32x4 d = ld128_stream(src + ((i + 3 * nthr) << 4));
        st128_stream(dst + (i << 4), a);
        st128_stream(dst + ((i + nthr) << 4), b);
        st128_stream(dst + ((i + 2 * nthr) << 4), c);
        st128_stream(dst + ((i + 3 * nthr) << 4), d);
    }
    for (; i < hi; i += nthr) st128_stream(dst + (i << 4), ld128_stream(src + (i << 4)));
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (tid < (nbytes & 15u)) dst[(nvec << 4) + tid] = src[(nvec << 4) + tid];
}

// Advances a launch epoch kept in device memory: 1, 2, ..., max_epoch, 1, ...
// and clears the staging memory whenever it starts over, so that no sector
// tag of an earlier launch with the same number survives.  With `track` the
// word behind the epoch remembers the protocol of the launch before
// (protocol + 1; 0 = none yet), and the memory is also cleared when an LL128
// launch follows a Simple one: raw payload a Simple launch left in a slot could
// pass for the sector tags an LL128 launch looks for.  The decision is taken
// here, on the device, when the kernel runs - not on the host when the launch
// is enqueued - so a launch that was captured into a graph decides anew at
// every replay.  One block: the clearing is rare.
__global__ void __launch_bounds__(1024) epoch_advance_kernel(uint32_t* epoch_word, uint8_t* staging,
                                                             uint64_t staging_bytes,
                                                             uint32_t max_epoch, uint32_t track,
                                                             uint32_t protocol) {
    const uint32_t cur = epoch_word[0];
    const uint32_t before = track ? epoch_word[1] : 0u;
    __syncthreads();
    uint32_t next = cur + 1u;
    const bool tags_forged = track && protocol == 0u /* LL128 */ && before == 2u /* Simple + 1 */;
    if (cur == 0u || cur >= max_epoch || tags_forged) {   // first use, tags about to repeat, or forgeable
        const u32x4 zero = {0u, 0u, 0u, 0u};
        for (uint64_t i = threadIdx.x; i < (staging_bytes >> 4); i += blockDim.x)
            *reinterpret_cast<u32x4*>(staging + (i << 4)) = zero;
        next = 1u;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        epoch_word[0] = next;
        if (track) epoch_word[1] = protocol + 1u;
    }
}

// Clears [p, p + nbytes), whole 16-byte vectors, with a grid-stride fill.  It
// stands where a memset on the stream would: a fill kernel can be captured
// into a HIP graph and replayed, a memset node cannot be relied on there.
__global__ void __launch_bounds__(256) zero_kernel(uint8_t* p, uint64_t nbytes) {
    const u32x4 zero = {0u, 0u, 0u, 0u};
    const uint64_t nvec = nbytes >> 4;
    const uint64_t nthr = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += nthr)
        *reinterpret_cast<u32x4*>(p + (i << 4)) = zero;
}

// Read-only pass: XOR of all whole 16-byte vectors of a buffer, folded into
// four 32-bit words (per wavefront by lane exchange, per block through LDS,
// then one atomic per word and block).  The HBM read-bandwidth yardstick: the
// ring kernels read far more than they write.
__global__ void __launch_bounds__(1024) read_xor_kernel(const uint8_t* __restrict__ src,
                                                        uint64_t nbytes, uint32_t* out) {
    __shared__ uint32_t part[16][4];
    const uint64_t nvec = nbytes >> 4;
    const uint64_t per = (nvec + gridDim.x - 1) / gridDim.x;
    const uint64_t lo = (uint64_t)blockIdx.x * per;
    const uint64_t hi = lo + per < nvec ? lo + per : nvec;
    const uint64_t nthr = blockDim.x;
    u32x4 acc = {0u, 0u, 0u, 0u};
    uint64_t i = lo + threadIdx.x;
    for (; i + 3 * nthr < hi; i += 4 * nthr) {
        u32x4 a = ld128_stream(src + (i << 4));
        u32x4 b = ld128_stream(src + ((i + nthr) << 4));
        u32x4 c = ld128_stream(src + ((i + 2 * nthr) << 4));
        u32x4 d = ld128_stream(src + ((i + 3 * nthr) << 4));
        acc ^= (a ^ b) ^ (c ^ d);
    }
    for (; i < hi; i += nthr) acc ^= ld128_stream(src + (i << 4));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        acc.x ^= __shfl_xor(acc.x, off);
        acc.y ^= __shfl_xor(acc.y, off);
        acc.z ^= __shfl_xor(acc.z, off);
        acc.w ^= __shfl_xor(acc.w, off);
    }
    const int wv = wave_in_block();
    if (lane_id() == 0) {
        part[wv][0] = acc.x; part[wv][1] = acc.y; part[wv][2] = acc.z; part[wv][3] = acc.w;
    }
    __syncthreads();
    if (threadIdx.x < 4) {
        uint32_t x = 0;
        const int nw = (int)(blockDim.x >> 6);
        for (int k = 0; k < nw; ++k) x ^= part[k][threadIdx.x];
        atomicXor(out + threadIdx.x, x);
    }
}

// ---- the memory traffic of a ring step, without the ring ---------------------
// Every wavefront runs `iters` steps; in a step it loads its own 960-byte block
// from `rows` the way the ring kernels do (streaming, flag lanes 4 bytes early),
// loads 1 KiB from one of its two private slots in `staging` with the loads
// the polls use, adds, and stores 1 KiB into the other slot - whichever of the
// three `what` selects.  Nobody waits for anybody: the launch takes what the
// device needs for that mix of accesses, the yardstick the ring kernels are
// measured against.
template <int WHAT>
__global__ void __launch_bounds__(256) step_mix_kernel(const uint8_t* __restrict__ rows,
                                                       uint8_t* staging, uint32_t staging_bytes,
                                                       uint32_t waves, uint32_t iters,
                                                       uint32_t* sink) {
    // WHAT & 8: the own-row load writes straight into LDS (buffer_load ... lds,
    // 16 bytes per lane) and the adder reads it from there
    __shared__ __attribute__((aligned(16))) uint8_t landing[(WHAT & 8) ? 4 * kBlockMsg : 16];
    const LaneMap m;
    const uint32_t wave = blockIdx.x * (blockDim.x >> 6) + (uint32_t)wave_in_block();
    if (wave >= waves) return;
    const Window win(staging, staging_bytes);
    const uint32_t slot0 = wave * 2u * kBlockMsg;
    MINT_LDS uint8_t* const mine = (MINT_LDS uint8_t*)landing +
                                   ((WHAT & 8) ? (uint32_t)wave_in_block() * kBlockMsg : 0u);
    u32x4 acc = {0u, 0u, 0u, 0u};
    for (uint32_t i = 0; i < iters; ++i) {
        u32x4 own = {0u, 0u, 0u, 0u}, got = {0u, 0u, 0u, 0u};
        if (WHAT & 2) got = ld128<CP_SC1>(win, slot0 + (i & 1u) * kBlockMsg + m.lane * 16u);
        if constexpr ((WHAT & 9) == 9) {
            const uint32_t off = m.flag_lane ? m.raw_off - 4u : m.raw_off;
            __builtin_amdgcn_global_load_lds(
                (MINT_GLOBAL const void*)(rows + (uint64_t)(i * waves + wave) * kBlockRawLL + off),
                (MINT_LDS void*)mine, 16, 0, /*nt*/ 2);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            own = *(MINT_LDS const u32x4*)(mine + m.lane * 16u);
        } else if (WHAT & 1) {
            own = ll_fetch_raw(rows, 0, i * waves + wave, true, m);
        }
        u32x4 x = add_rn<DT_F16>(own, got);
        // WHAT >> 8: that many times sixteen scalar additions between the
        // loads and the store - the bookkeeping of a ring step without the
        // ring (a compute unit has one scalar unit for all its wavefronts)
        if constexpr ((WHAT >> 8) != 0) {
            uint32_t busy = __builtin_amdgcn_readfirstlane(x.x);
#pragma unroll
            for (int k = 0; k < (WHAT >> 8) * 16; ++k)
                asm volatile("s_add_u32 %0, %0, 1" : "+s"(busy) : : "scc");
            x.x ^= busy & 0u;
        }
        // WHAT & 16: the block also goes back to HBM, as a copying position
        // saves what it received (a streaming store of the 960 raw bytes)
        if (WHAT & 16)
            ll_save_raw(const_cast<uint8_t*>(rows), (uint64_t)waves * iters * kBlockRawLL,
                        i * waves + wave, true, m, x);
        if (WHAT & 4) st128<CP_NONE>(win, slot0 + ((i + 1u) & 1u) * kBlockMsg + m.lane * 16u, x);
        else if (!(WHAT & 16)) acc ^= x;
    }
    if (!(WHAT & 20) && acc.x == 0x9E3779B9u && acc.y == 0x85EBCA6Bu && acc.z == 0xC2B2AE35u)
        sink[0] = acc.w;     // keeps the loads alive; practically never taken
}

// ---- the same traffic with several steps in flight per wavefront ---------------
// step_mix_kernel above has one step in flight per wavefront: a step's loads
// are issued, waited for, added and stored before the next step's loads go
// out, and since a wavefront's vector-memory operations retire in issue order
// every step also waits for the previous step's store.  Its time is therefore
// (steps) x (a load's latency + a store's), which need not be what the device
// can do with the mix.  Here the loads run AHEAD steps ahead of their use and
// are older than the store of the step before them, so a wait for a step's
// loads leaves the younger loads and every store in flight: AHEAD + 1 steps of
// loads per wavefront, no store -> load chain inside a wavefront.
// A wavefront owns AHEAD + 2 slots of 1 KiB; it stores step i into its slot
// i mod (AHEAD + 2) and loads step j from slot (j + 1) mod (AHEAD + 2) of its
// *partner* - the same wavefront of the thread block 8 further on (block ^ 8:
// the same XCD, another CU), or itself (partner = 0) - which is what a ring
// does to a line: written by one CU, read by another a step later.  Nothing is
// synchronised; the values are whatever is there.
//
// The order of the memory operations is what is measured: a compiler fence and
// a scheduling barrier stand between the phases of a step (the compiler, left
// to itself, gathers the loads of an unrolled loop at its top and waits for
// all of them); the waits are the compiler's own, which counts the operations
// issued after the one it needs.
__device__ __forceinline__ void mix_phase() {
    compiler_fence();
    __builtin_amdgcn_sched_barrier(0);
    compiler_fence();
}
template <int WHAT, int AHEAD>
__global__ void __launch_bounds__(256) step_mix_deep_kernel(const uint8_t* rows, uint8_t* staging,
                                                            uint32_t staging_bytes,
                                                            uint32_t waves, uint32_t iters,
                                                            uint32_t partner, uint32_t* sink) {
    constexpr uint32_t NS = AHEAD + 2;
    const LaneMap m;
    const uint32_t wpb = blockDim.x >> 6;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(blockIdx.x * wpb + (uint32_t)wave_in_block());
    if (wave >= waves) return;
    uint32_t other = partner ? wave ^ (8u * wpb) : wave;
    if (other >= waves) other = wave;
    const Window win(staging, staging_bytes);
    const uint32_t st_base = wave * NS * kBlockMsg + m.lane * 16u;
    const uint32_t ld_base = other * NS * kBlockMsg + m.lane * 16u;
    const uint32_t row_lane = m.flag_lane ? m.raw_off - 4u : m.raw_off;
    u32x4 own[AHEAD + 1], got[AHEAD + 1];
    u32x4 acc = {0u, 0u, 0u, 0u};
    uint32_t ld_slot = 1u, st_slot = 0u, ld_step = 0u;
    // loads of one step; beyond the last step any valid address
    auto issue = [&](int d) __attribute__((always_inline)) {
        const uint32_t j = ld_step < iters ? ld_step : iters - 1u;
        own[d] = got[d] = u32x4{0u, 0u, 0u, 0u};
        if (WHAT & 1)
            own[d] = __builtin_nontemporal_load((MINT_GLOBAL const u32x4_a1*)(
                rows + (uint64_t)(j * waves + wave) * kBlockRawLL + row_lane));
        if (WHAT & 2) got[d] = ld128<CP_SC1>(win, ld_base + ld_slot * kBlockMsg);
        ld_slot = ld_slot + 1u == NS ? 0u : ld_slot + 1u;
        ++ld_step;
    };
    // the prologue leaves the queue a later step finds (a store behind every
    // step's loads): the compiler takes the smaller count where paths meet
#pragma unroll
    for (int d = 0; d <= AHEAD; ++d) {
        if (WHAT & 4) st128<CP_NONE>(win, st_base + (uint32_t)d * kBlockMsg, acc);
        mix_phase();
        issue(d);
        mix_phase();
    }
    for (uint32_t i = 0; i < iters; i += AHEAD + 1) {
#pragma unroll
        for (int d = 0; d <= AHEAD; ++d) {
            // (the store first: the step's registers are free again when the
            // loads that refill them are issued.  Either way the store is
            // younger than the loads the next wait is for.)
            const u32x4 x = add_rn<DT_F16>(own[d], got[d]);
            mix_phase();
            if (WHAT & 4) st128<CP_NONE>(win, st_base + st_slot * kBlockMsg, x);
            else acc ^= x;
            st_slot = st_slot + 1u == NS ? 0u : st_slot + 1u;
            mix_phase();
            issue(d);
            mix_phase();
        }
    }
    if (!(WHAT & 4) && acc.x == 0x9E3779B9u && acc.y == 0x85EBCA6Bu && acc.z == 0xC2B2AE35u)
        sink[0] = acc.w;     // keeps the loads alive; practically never taken
}

// ---- LL128 codec, wave64 layout: one wavefront per block -------------------
__global__ void __launch_bounds__(256) pack_wave64_kernel(const uint8_t* __restrict__ raw,
                                                          uint8_t* __restrict__ msg,
                                                          uint64_t nbytes, uint32_t nblocks,
                                                          uint64_t flag_base, uint64_t flag_stride) {
    const LaneMap m;
    const uint32_t waves = gridDim.x * (blockDim.x >> 6);
    const uint32_t wave = blockIdx.x * (blockDim.x >> 6) + (uint32_t)wave_in_block();
    for (uint32_t g = wave; g < nblocks; g += waves) {
        u32x4 v = ll_load_raw(raw, nbytes, g, m);
        // line = two sectors; both carry the low 32 bits of the line's flag
        const uint64_t flag = flag_base + ((uint64_t)g * 8u + (m.sector >> 1)) * flag_stride;
        if (m.flag_lane) v.w = (uint32_t)flag;
        *reinterpret_cast<u32x4*>(msg + (uint64_t)g * kBlockMsg + m.lane * 16u) = v;
    }
}
__global__ void __launch_bounds__(256) unpack_wave64_kernel(const uint8_t* __restrict__ msg,
                                                            uint8_t* __restrict__ raw,
                                                            uint64_t nbytes, uint32_t nblocks,
                                                            uint64_t flag_base,
                                                            uint64_t flag_stride,
                                                            unsigned long long* bad_flags) {
    const LaneMap m;
    const uint32_t waves = gridDim.x * (blockDim.x >> 6);
    const uint32_t wave = blockIdx.x * (blockDim.x >> 6) + (uint32_t)wave_in_block();
    uint32_t bad = 0;
    for (uint32_t g = wave; g < nblocks; g += waves) {
        u32x4 v = *reinterpret_cast<const u32x4*>(msg + (uint64_t)g * kBlockMsg + m.lane * 16u);
        const uint64_t flag = flag_base + ((uint64_t)g * 8u + (m.sector >> 1)) * flag_stride;
        // a line is bad if either of its two sector tags is: pair up the
        // flag lanes of a line through the ballot, count once per line
        const uint64_t wrong = __ballot(m.flag_lane && v.w != (uint32_t)flag);
        for (uint32_t j = 0; j < 8u; ++j) bad += ((wrong >> (8u * j)) & 0xFFull) ? 1u : 0u;
        ll_save_raw(raw, nbytes, g, m, v);
    }
    if (bad && bad_flags && lane_id() == 0) atomicAdd(bad_flags, (unsigned long long)bad);
}

// ---- LL128 codec, reference pair layout: one thread per 16-byte message
// lane, 8 threads per line, exactly the reference's lane roles
// (protocol.py:57-100,132-137).
__device__ __forceinline__ void pair_lane(uint64_t t, uint64_t& line, uint32_t& k,
                                          uint64_t& raw_off, uint32_t& raw_len) {
    line = t >> 3;
    k = (uint32_t)(t & 7u);
    const uint64_t pair_base = (line >> 1) * 240u;
    const bool second = line & 1u;
    if (k != 7u) { raw_off = pair_base + (second ? 128u : 0u) + k * 16u; raw_len = 16u; }
    else         { raw_off = pair_base + (second ? 120u : 112u);         raw_len = 8u; }
}
__global__ void __launch_bounds__(256) pack_pair_kernel(const uint8_t* __restrict__ raw,
                                                        uint8_t* __restrict__ msg,
                                                        uint64_t nbytes, uint64_t nlines,
                                                        uint64_t flag_base, uint64_t flag_stride) {
    const uint64_t nthr = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; t < nlines * 8u; t += nthr) {
        uint64_t line, raw_off; uint32_t k, raw_len;
        pair_lane(t, line, k, raw_off, raw_len);
        u32x4 v = load_guarded(raw, raw_off, raw_len, nbytes);
        if (k == 7u) {
            const uint64_t flag = flag_base + line * flag_stride;
            v.z = (uint32_t)flag; v.w = (uint32_t)(flag >> 32);
        }
        *reinterpret_cast<u32x4*>(msg + (t << 4)) = v;
    }
}
__global__ void __launch_bounds__(256) unpack_pair_kernel(const uint8_t* __restrict__ msg,
                                                          uint8_t* __restrict__ raw,
                                                          uint64_t nbytes, uint64_t nlines,
                                                          uint64_t flag_base, uint64_t flag_stride,
                                                          unsigned long long* bad_flags) {
    const uint64_t nthr = (uint64_t)gridDim.x * blockDim.x;
    uint32_t bad = 0;
    for (uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; t < nlines * 8u; t += nthr) {
        uint64_t line, raw_off; uint32_t k, raw_len;
        pair_lane(t, line, k, raw_off, raw_len);
        u32x4 v = *reinterpret_cast<const u32x4*>(msg + (t << 4));
        if (k == 7u) {
            const uint64_t flag = flag_base + line * flag_stride;
            if (v.z != (uint32_t)flag || v.w != (uint32_t)(flag >> 32)) ++bad;
        }
        store_guarded(raw, raw_off, raw_len, nbytes, v);
    }
    if (bad && bad_flags) atomicAdd(bad_flags, (unsigned long long)bad);
}

// ---- out = rn(a + b) ------------------------------------------------------
template <int DT>
__global__ void __launch_bounds__(256) sum_kernel(const uint8_t* __restrict__ a,
                                                  const uint8_t* __restrict__ b,
                                                  uint8_t* __restrict__ out, uint64_t nbytes) {
    const uint64_t nvec = nbytes >> 4;
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint64_t nthr = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = tid; i < nvec; i += nthr) {
        u32x4 x = *reinterpret_cast<const u32x4*>(a + (i << 4));
        u32x4 y = *reinterpret_cast<const u32x4*>(b + (i << 4));
        *reinterpret_cast<u32x4*>(out + (i << 4)) = add_rn<DT>(x, y);
    }
    if (tid == 0 && (nbytes & 15u)) {
        u32x4 x = load_guarded(a, nvec << 4, 16u, nbytes);
        u32x4 y = load_guarded(b, nvec << 4, 16u, nbytes);
        store_guarded(out, nvec << 4, 16u, nbytes, add_rn<DT>(x, y));
    }
}

// ---- block -> XCD map -------------------------------------------------------
__global__ void xcd_map_kernel(uint32_t* out) {
    if (threadIdx.x == 0) out[blockIdx.x] = (uint32_t)xcc_id();
}

// ---- torn-line probe --------------------------------------------------------
// The payload of a sector is a function of its tag, so a consumer that sees
// the tag can tell whether the other bytes belong to it.  `per_sector` = 1 is
// the format the ring kernels use (a tag in every 64-byte sector, all 16
// tested); `per_sector` = 0 tests only the tag of the second sector of each
// 128-byte line, which is what a one-flag-per-line format amounts to.
__device__ __forceinline__ uint32_t probe_word(uint32_t tag, uint32_t lane, uint32_t d) {
    return (tag * 2654435761u) ^ (lane * 0x9E3779B1u + d * 0x85EBCA77u + 0x1234567u);
}
constexpr uint32_t kProbeDepth = 4;   // blocks per pair, reused round-robin

template <int LDCP, int STCP>
__global__ void __launch_bounds__(256) torn_probe_kernel(uint8_t* staging, uint32_t pairs,
                                                         uint32_t iters, int placement,
                                                         int per_sector, uint32_t epoch,
                                                         uint32_t budget,
                                                         unsigned long long* counters) {
    const LaneMap m;
    const uint32_t wpb = blockDim.x >> 6;
    uint32_t pb; bool producer;
    if (placement == 1) {
        // producer and consumer of a pair are consecutive blocks of the same XCD
        const uint32_t xcd = blockIdx.x % 8u, y = blockIdx.x / 8u;
        pb = (y >> 1) * 8u + xcd;
        producer = !(y & 1u);
    } else {
        pb = blockIdx.x >> 1;
        producer = !(blockIdx.x & 1u);
    }
    const uint32_t pair = pb * wpb + (uint32_t)wave_in_block();
    if (pair >= pairs) return;
    const uint32_t data_bytes = pairs * kProbeDepth * kBlockMsg;
    const Window win(staging, data_bytes);
    uint64_t* tail = reinterpret_cast<uint64_t*>(staging + data_bytes + (uint64_t)pair * 128u);
    const uint64_t flag_hi = (uint64_t)epoch << 32;
    unsigned long long checked = 0, torn = 0, polls = 0, timeouts = 0, first_half = 0;
    for (uint32_t t = 0; t < iters; ++t) {
        const uint32_t off = (pair * kProbeDepth + t % kProbeDepth) * kBlockMsg;
        const uint32_t tag = (epoch << 20) | ((t + 1u) & 0xFFFFFu);
        if (producer) {
            if (t >= kProbeDepth) {
                bool ok = false;
                for (uint32_t spins = 0; spins <= budget; ++spins) {
                    uint64_t v = ld64_agent(tail);
                    uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
                    uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
                    if (hi == epoch && lo >= t - kProbeDepth + 1) { ok = true; break; }
                    __builtin_amdgcn_s_sleep(1);
                }
                if (!ok) { ++timeouts; break; }
            }
            u32x4 v = {probe_word(tag, m.lane, 0), probe_word(tag, m.lane, 1),
                       probe_word(tag, m.lane, 2), probe_word(tag, m.lane, 3)};
            ll_send<STCP>(win, off, v, tag, m);
        } else {
            u32x4 v; bool ok = false;
            for (uint32_t spins = 0; spins <= budget; ++spins) {
                compiler_fence();
                ++polls;
                v = ld128<LDCP>(win, off + m.lane * 16u);
                const bool tested = m.flag_lane && (per_sector || (m.sector & 1u));
                if (wave_all(!tested || v.w == tag)) { ok = true; break; }
                __builtin_amdgcn_s_sleep(1);
            }
            if (!ok) { ++timeouts; break; }
            bool bad = v.x != probe_word(tag, m.lane, 0) || v.y != probe_word(tag, m.lane, 1) ||
                       v.z != probe_word(tag, m.lane, 2);
            bad = bad || (m.flag_lane ? v.w != tag : v.w != probe_word(tag, m.lane, 3));
            const uint64_t mask = __ballot(bad);
            for (uint32_t j = 0; j < 8u; ++j) {
                const uint32_t line = (uint32_t)(mask >> (8u * j)) & 0xFFu;
                torn += line ? 1u : 0u;
                first_half += line == 0x0Fu ? 1u : 0u;   // exactly the first sector stale
            }
            checked += 8u;
            if (lane_id() == 0) {
                if (STCP == CP_NONE) st64_local(tail, flag_hi | (uint64_t)(t + 1));
                else st64_agent(tail, flag_hi | (uint64_t)(t + 1));
            }
        }
    }
    if (lane_id() == 0) {
        if (checked) atomicAdd(counters + 0, checked);
        if (torn) atomicAdd(counters + 1, torn);
        if (polls) atomicAdd(counters + 2, polls);
        if (timeouts) atomicAdd(counters + 3, timeouts);
        if (first_half) atomicAdd(counters + 4, first_half);
    }
}

}  // namespace mint
