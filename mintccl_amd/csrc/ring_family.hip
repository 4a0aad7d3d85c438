// The ring kernels of one element type (MINT_FAMILY_DT: 0 f16, 1 bf16, 2 f32,
// 3 bytes) and their launcher.
#include <atomic>

#include "ring_launch.hpp"

#ifndef MINT_FAMILY_DT
#error "compile with -DMINT_FAMILY_DT=0..3"
#endif

namespace mint {
namespace {

template <int PROTO, int DT, int CP>
int launch_ring_u(const Plan& plan, hipStream_t stream) {
    void (*kernel)(const RingArgs) = nullptr;
    switch (plan.unroll) {
        case 4: kernel = ring_kernel<PROTO, DT, CP, 4>; break;
        case 2: kernel = ring_kernel<PROTO, DT, CP, 2>; break;
        default: kernel = ring_kernel<PROTO, DT, CP, 1>; break;
    }
    // Every wavefront of the launch polls words other wavefronts write, so
    // the whole grid has to be resident at once.  The occupancy of a kernel
    // at a block size does not change: ask once (per block size) and keep it.
    // (these statics are per template instantiation, i.e. per kernel family)
    static std::atomic<int> cached[3][9] = {};       // [unroll][threads / 64]
    static std::atomic<int> cus{0};
    std::atomic<int>& memo = cached[plan.unroll == 4 ? 2 : (plan.unroll == 2 ? 1 : 0)]
                                   [plan.threads / 64];
    int per_cu = memo.load(std::memory_order_relaxed);
    if (per_cu == 0) {
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, plan.threads, 0) !=
            hipSuccess)
            return MINT_ERR_HIP;
        // Count one wavefront per SIMD less than the query allows.  Measured:
        // at 4 waves per block the query says 7 blocks per CU, yet from 6
        // blocks per CU on the grid is no longer dealt out in one go and a
        // launch takes a third longer (the query does not see the scalar
        // registers the platform sets aside per wave for its trap handler;
        // a build squeezed into 16 fewer registers moved the step by exactly
        // one wave per SIMD).
        const int waves_per_block = plan.threads / 64;
        per_cu = (per_cu * waves_per_block - 4) / waves_per_block;
        if (per_cu < 1) per_cu = 1;
        memo.store(per_cu, std::memory_order_relaxed);
    }
    int ncu = cus.load(std::memory_order_relaxed);
    if (ncu == 0) { ncu = device_cus(); cus.store(ncu, std::memory_order_relaxed); }
    if (plan.blocks > per_cu * ncu) return MINT_ERR_RESIDENCY;
    hipLaunchKernelGGL(kernel, dim3((unsigned)plan.blocks), dim3((unsigned)plan.threads), 0, stream,
                       plan.args);
    return launch_status();
}

template <int PROTO, int DT>
int launch_ring_cp(const Plan& plan, int cache_policy, hipStream_t stream) {
    switch (cache_policy) {
        case 0: return launch_ring_u<PROTO, DT, 0>(plan, stream);
        case 1: return launch_ring_u<PROTO, DT, 1>(plan, stream);
        default: return launch_ring_u<PROTO, DT, 2>(plan, stream);
    }
}

template <int DT>
int launch_family(const Plan& plan, int protocol, int cache_policy, hipStream_t stream) {
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
