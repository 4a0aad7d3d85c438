// The ring kernels of one element type (MINT_FAMILY_DT: 0 f16, 1 bf16, 2 f32,
// 3 bytes) and their launcher.
#include <atomic>

#include "hypercube.hpp"
#include "ring_launch.hpp"
#include "temporal.hpp"
#include "tree.hpp"

#ifndef MINT_FAMILY_DT
#error "compile with -DMINT_FAMILY_DT=0..3"
#endif

namespace mint {
namespace {

// Thread blocks of `threads` threads (and `lds_bytes` of LDS) that a CU holds
// at once.  Every wavefront of a ring launch polls words other wavefronts
// write, so the whole grid has to be resident.  The occupancy query is asked
// twice: for the block size, and for blocks of one wavefront, which tells how
// many wavefronts of this kernel a CU takes.  Of those at most 6 per SIMD are
// counted.  Measured: where the query says 7 (the kernels need 98 - 106
// scalar registers), a grid of 6 blocks of 4 wavefronts per CU runs in one go
// and one of 7 takes a third longer - the query does not see the scalar
// registers the platform sets aside per wavefront for its trap handler (a
// build squeezed into 16 fewer registers moved the step by exactly one
// wavefront per SIMD).
template <typename Kernel>
int resident_blocks_per_cu(Kernel kernel, int threads, size_t lds_bytes) {
    int per_cu = 0, waves_per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, lds_bytes) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&waves_per_cu, kernel, 64, 0) != hipSuccess)
        return -1;
    if (waves_per_cu > 24) waves_per_cu = 24;
    const int by_waves = waves_per_cu / (threads / 64);
    if (by_waves < per_cu) per_cu = by_waves;
    return per_cu < 1 ? 1 : per_cu;
}

// Blocks of `kernel` the current device holds at once.  The occupancy of a
// kernel at a block size does not change, so it is asked once - per device: a
// process may drive several, and they need not be alike.  `memo` holds one
// entry per device (0 = not asked yet).  Negative on failure.
constexpr int kMemoDevices = 64;
template <typename Kernel>
int resident_capacity(Kernel kernel, int threads, size_t lds_bytes, std::atomic<int>* memo) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMemoDevices) return -1;
    int per_cu = memo[dev].load(std::memory_order_relaxed);
    if (per_cu == 0) {
        per_cu = resident_blocks_per_cu(kernel, threads, lds_bytes);
        if (per_cu < 0) return -1;
        memo[dev].store(per_cu, std::memory_order_relaxed);
    }
    static std::atomic<int> cus[kMemoDevices] = {};
    int ncu = cus[dev].load(std::memory_order_relaxed);
    if (ncu == 0) {
        ncu = device_cus();
        cus[dev].store(ncu, std::memory_order_relaxed);
    }
    return per_cu * ncu;
}

// Launch a plan whose grid fits `capacity` blocks.  Compute units set apart for
// origins need a larger grid (blocks with nothing to do fill the rounds): where
// that one does not fit and the plain one does, the plain order runs.
inline int launch_resident(void (*kernel)(const RingArgs), const Plan& plan, int capacity,
                           hipStream_t stream) {
    if (plan.blocks <= capacity) {
        hipLaunchKernelGGL(kernel, dim3((unsigned)plan.blocks), dim3((unsigned)plan.threads), 0, stream,
                           plan.args);
        return launch_status();
    }
    if (!plan.args.origin_cus || plan.blocks_plain > capacity) return MINT_ERR_RESIDENCY;
    RingArgs plain = plan.args;
    plain.origin_cus = 0;
    hipLaunchKernelGGL(kernel, dim3((unsigned)plan.blocks_plain), dim3((unsigned)plan.threads), 0,
                       stream, plain);
    return launch_status();
}

// Own rows through LDS (reducing element types only): WPB wave-channels and
// one fetcher wavefront per thread block, R groups in flight per wave-channel.
template <int DT, int CP>
int launch_ring_lds(const Plan& plan, hipStream_t stream) {
    if constexpr (DT == DT_BYTES) {
        return MINT_ERR_ARG;
    } else {
        const int wpb = plan.threads / 64;
        void (*kernel)(const RingArgs) = nullptr;
        if (wpb == 4)
            kernel = plan.unroll == 2 ? ring_kernel_lds<DT, CP, 2, 4, 2> : ring_kernel_lds<DT, CP, 1, 4, 3>;
        else
            kernel = plan.unroll == 2 ? ring_kernel_lds<DT, CP, 2, 7, 1> : ring_kernel_lds<DT, CP, 1, 7, 2>;
        const int threads = plan.threads + 64;
        const size_t lds_bytes = kLdsHeader + (size_t)wpb * plan.args.fetch_depth *
                                                  (size_t)plan.unroll * kBlockMsg;
        static std::atomic<int> cached[2][2][kMemoDevices] = {};   // [wpb == 7][unroll == 2][device]
        const int capacity = resident_capacity(kernel, threads, lds_bytes,
                                               cached[wpb == 7][plan.unroll == 2]);
        if (capacity < 0) return MINT_ERR_HIP;
        if (plan.blocks > capacity) return MINT_ERR_RESIDENCY;
        hipLaunchKernelGGL(kernel, dim3((unsigned)plan.blocks), dim3((unsigned)threads), lds_bytes,
                           stream, plan.args);
        return launch_status();
    }
}

template <int PROTO, int DT, int CP>
int launch_ring_u(const Plan& plan, hipStream_t stream) {
    if (plan.lds) return launch_ring_lds<DT, CP>(plan, stream);
    void (*kernel)(const RingArgs) = nullptr;
    switch (plan.unroll) {
        case 4: kernel = ring_kernel<PROTO, DT, CP, 4>; break;
        case 2: kernel = ring_kernel<PROTO, DT, CP, 2>; break;
        default: kernel = ring_kernel<PROTO, DT, CP, 1>; break;
    }
    // (These statics are per template instantiation, i.e. per kernel family.)
    static std::atomic<int> cached[3][9][kMemoDevices] = {};   // [unroll][threads / 64][device]
    const int capacity = resident_capacity(
        kernel, plan.threads, 0,
        cached[plan.unroll == 4 ? 2 : (plan.unroll == 2 ? 1 : 0)][plan.threads / 64]);
    if (capacity < 0) return MINT_ERR_HIP;
    return launch_resident(kernel, plan, capacity, stream);
}

template <int PROTO, int DT>
int launch_ring_cp(const Plan& plan, int cache_policy, hipStream_t stream) {
    switch (cache_policy) {
        case 0: return launch_ring_u<PROTO, DT, 0>(plan, stream);
        case 1: return launch_ring_u<PROTO, DT, 1>(plan, stream);
        default: return launch_ring_u<PROTO, DT, 2>(plan, stream);
    }
}

// Broadcast / reduce over a binary tree (LL128): one wavefront per (node,
// wave-channel), all of them resident like a ring's.
template <int DT, int CP>
int launch_tree(const Plan& plan, hipStream_t stream) {
    void (*kernel)(const RingArgs) = tree_kernel<DT, CP>;
    static std::atomic<int> cached[9][kMemoDevices] = {};      // [threads / 64][device]
    const int capacity = resident_capacity(kernel, plan.threads, 0, cached[plan.threads / 64]);
    if (capacity < 0) return MINT_ERR_HIP;
    return launch_resident(kernel, plan, capacity, stream);
}

// Reduce-scatter / allgather over a hypercube (LL128): one wavefront per (row,
// node, wave-channel), all of them resident like a ring's.
template <int DT, int CP>
int launch_hyper(const Plan& plan, hipStream_t stream) {
    void (*kernel)(const RingArgs) = hyper_kernel<DT, CP>;
    static std::atomic<int> cached[9][kMemoDevices] = {};      // [threads / 64][device]
    const int capacity = resident_capacity(kernel, plan.threads, 0, cached[plan.threads / 64]);
    if (capacity < 0) return MINT_ERR_HIP;
    return launch_resident(kernel, plan, capacity, stream);
}

// Allgather, temporal schedule (LL128, bytes): one wavefront per (rank,
// wave-channel).
template <int CP>
int launch_temporal(const Plan& plan, hipStream_t stream) {
    void (*kernel)(const RingArgs) = temporal_kernel<CP>;
    static std::atomic<int> cached[9][kMemoDevices] = {};      // [threads / 64][device]
    const int capacity = resident_capacity(kernel, plan.threads, 0, cached[plan.threads / 64]);
    if (capacity < 0) return MINT_ERR_HIP;
    return launch_resident(kernel, plan, capacity, stream);
}

template <int DT>
int launch_family(const Plan& plan, int protocol, int cache_policy, hipStream_t stream) {
    if (plan.args.op == OP_ALLGATHER_TEMPORAL) {
        if constexpr (DT == DT_BYTES) {
            switch (cache_policy) {
                case 0: return launch_temporal<0>(plan, stream);
                case 1: return launch_temporal<1>(plan, stream);
                default: return launch_temporal<2>(plan, stream);
            }
        } else {
            return MINT_ERR_ARG;
        }
    }
    if (plan.args.op == OP_HYPER_REDUCESCATTER || plan.args.op == OP_HYPER_ALLGATHER) {
        switch (cache_policy) {
            case 0: return launch_hyper<DT, 0>(plan, stream);
            case 1: return launch_hyper<DT, 1>(plan, stream);
            default: return launch_hyper<DT, 2>(plan, stream);
        }
    }
    if (plan.args.op == OP_TREE_BROADCAST || plan.args.op == OP_TREE_REDUCE) {
        switch (cache_policy) {
            case 0: return launch_tree<DT, 0>(plan, stream);
            case 1: return launch_tree<DT, 1>(plan, stream);
            default: return launch_tree<DT, 2>(plan, stream);
        }
    }
    return protocol == MINT_PROTO_LL128 ? launch_ring_cp<PROTO_LL128, DT>(plan, cache_policy, stream)
                                        : launch_ring_cp<PROTO_SIMPLE, DT>(plan, cache_policy, stream);
}

}  // namespace

#if MINT_FAMILY_DT == 0
int launch_ring_family_f16(const Plan& plan, int protocol, int cache_policy, hipStream_t stream) {
    return launch_family<DT_F16>(plan, protocol, cache_policy, stream);
}
#elif MINT_FAMILY_DT == 1
int launch_ring_family_bf16(const Plan& plan, int protocol, int cache_policy, hipStream_t stream) {
    return launch_family<DT_BF16>(plan, protocol, cache_policy, stream);
}
#elif MINT_FAMILY_DT == 2
int launch_ring_family_f32(const Plan& plan, int protocol, int cache_policy, hipStream_t stream) {
    return launch_family<DT_F32>(plan, protocol, cache_policy, stream);
}
#else
int launch_ring_family_bytes(const Plan& plan, int protocol, int cache_policy, hipStream_t stream) {
    return launch_family<DT_BYTES>(plan, protocol, cache_policy, stream);
}
#endif

}  // namespace mint
