// Host side of the ring kernels: the launch plan and one launcher per element
// type.  Each launcher lives in a translation unit of its own (ring_family.hip
// compiled with MINT_FAMILY_DT = 0..3), which lets the build compile the four
// kernel families in parallel.
#pragma once
#include <hip/hip_runtime.h>

#include "../../include/mintccl.h"
#include "ring.hpp"

namespace mint {

struct Plan {
    RingArgs args;
    int blocks, threads, unroll;
    int blocks_plain;         // the grid without CUs set apart for origins (args.origin_cus)
    size_t staging_need;      // bytes of staging per rank: slots + credit words
    bool empty;
    bool lds;                 // own rows through LDS: `threads` counts the wave-channels'
                              // threads only, the launch adds the fetcher wavefront
};

inline int launch_status() { return hipGetLastError() == hipSuccess ? MINT_OK : MINT_ERR_HIP; }

inline int device_cus() {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
        return 0;
    return cus;
}

// protocol: MINT_PROTO_*; cache_policy: 0 agent, 1 system, 2 XCD-local
int launch_ring_family_f16(const Plan& plan, int protocol, int cache_policy, hipStream_t stream);
int launch_ring_family_bf16(const Plan& plan, int protocol, int cache_policy, hipStream_t stream);
int launch_ring_family_f32(const Plan& plan, int protocol, int cache_policy, hipStream_t stream);
int launch_ring_family_bytes(const Plan& plan, int protocol, int cache_policy, hipStream_t stream);

}  // namespace mint
