// Device primitives for gfx950 (CDNA4, 64-lane wavefronts).
//
// These stand where the reference keeps PTX strings (primitive.py:22-247):
//   thread_id        (primitive.py:22-34)   -> lane_id / wave_in_block
//   any_sync         (primitive.py:88-103)  -> wave_all / wave_any (64-bit ballot)
//   load128/store128 (primitive.py:180-203) -> ld128 / st128 with a cache policy
//   load64/store64   (primitive.py:205-227) -> ld64_agent / st64_agent
//   SumFP16          (primitive.py:232-247) -> add_rn<DT_F16>, plus bf16 and f32
//
// The reference's ld/st are "volatile": they bypass L1 and that is all it
// needs, because each of its ranks is a GPU of its own.  Here producer and
// consumer are workgroups of one GPU, possibly on different XCDs with their own
// L2, so every access to staging memory carries explicit scope bits:
//   sc1        agent scope  - misses the per-CU vector L1 and the non-coherent
//                             part of the per-XCD L2; stores write through
//   sc0 sc1    system scope
//   nt         non-temporal - streaming hint for data that is touched once
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mint {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

enum : int { DT_F16 = 0, DT_BF16 = 1, DT_F32 = 2, DT_BYTES = 3 };

// Cache-policy operand of the buffer instructions on gfx94x/gfx950.
enum : int { CP_NONE = 0, CP_SC0 = 1, CP_NT = 2, CP_SC1 = 16,
             CP_AGENT = CP_SC1, CP_SYSTEM = CP_SC0 | CP_SC1 };

__device__ __forceinline__ int lane_id() { return (int)(threadIdx.x & 63u); }
__device__ __forceinline__ int wave_in_block() { return (int)(threadIdx.x >> 6); }

// XCD the wave runs on (XCC_ID hardware register, bits 3:0).
__device__ __forceinline__ int xcc_id() {
    return (int)__builtin_amdgcn_s_getreg(20 | (0 << 6) | (3 << 11));
}

__device__ __forceinline__ bool wave_all(bool p) { return __ballot(p) == ~0ull; }
__device__ __forceinline__ bool wave_any(bool p) { return __ballot(p) != 0ull; }

// Keeps the compiler from hoisting or merging memory accesses across this
// point; emits no instruction.
__device__ __forceinline__ void compiler_fence() { asm volatile("" ::: "memory"); }

// A window of up to 4 GiB of device memory addressed with 32-bit offsets
// through the buffer instructions.  Accesses beyond `bytes` read zero and
// drop stores, which is what keeps a mis-sized launch from faulting.
struct Window {
    __amdgpu_buffer_rsrc_t rsrc;
    __device__ __forceinline__ Window(const void* base, uint32_t bytes)
        : rsrc(__builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes,
                                                 0x00020000)) {}
};

template <int CP>
__device__ __forceinline__ u32x4 ld128(const Window& w, uint32_t off) {
    return __builtin_amdgcn_raw_buffer_load_b128(w.rsrc, (int)off, 0, CP);
}
template <int CP>
__device__ __forceinline__ void st128(const Window& w, uint32_t off, u32x4 v) {
    __builtin_amdgcn_raw_buffer_store_b128(v, w.rsrc, (int)off, 0, CP);
}
// A load with a wave-uniform part of the offset in a scalar register (the
// instruction adds it): what changes from step to step costs no vector add.
// Loads only.  A 128-bit store with its offset in a scalar register was seen
// to pick up the next vector instruction's write to its first data register
// (word 0 of lanes 12 - 15 of every 16, now and then): the compiler leaves no
// gap after such a store, which it does after one with a constant offset.
template <int CP>
__device__ __forceinline__ u32x4 ld128(const Window& w, uint32_t off, uint32_t uniform_off) {
    return __builtin_amdgcn_raw_buffer_load_b128(w.rsrc, (int)off, (int)uniform_off, CP);
}
template <int CP>
__device__ __forceinline__ u32x2 ld64(const Window& w, uint32_t off) {
    return __builtin_amdgcn_raw_buffer_load_b64(w.rsrc, (int)off, 0, CP);
}
template <int CP>
__device__ __forceinline__ void st64(const Window& w, uint32_t off, u32x2 v) {
    __builtin_amdgcn_raw_buffer_store_b64(v, w.rsrc, (int)off, 0, CP);
}

// Pointers into device memory are cast to the global address space before
// use: a generic pointer makes the compiler emit flat_* instructions, which
// count on two wait counters at once and so tie vector-memory waits to
// scalar/LDS ones.
#define MINT_GLOBAL __attribute__((address_space(1)))
#define MINT_LDS __attribute__((address_space(3)))
template <typename T>
__device__ __forceinline__ MINT_GLOBAL T* as_global(T* p) {
    return (MINT_GLOBAL T*)p;
}

// 64-bit words shared between workgroups (credits, status): relaxed atomics
// at agent scope compile to global_load/store_dwordx2 ... sc1.
__device__ __forceinline__ uint64_t ld64_agent(const uint64_t* p) {
    return __hip_atomic_load(as_global(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st64_agent(uint64_t* p, uint64_t v) {
    __hip_atomic_store(as_global(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Plain 64-bit store (no scope bits): stays in the L2 of the XCD that runs the
// wave.  Relaxed atomic at wavefront scope, so the compiler keeps it whole and
// in program order with respect to other atomics.
__device__ __forceinline__ void st64_local(uint64_t* p, uint64_t v) {
    __hip_atomic_store(as_global(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
}
// A 64-bit word read through the scalar unit, past the scalar cache (glc), from
// the L2 of the XCD the wave runs on.  Scalar loads count on lgkmcnt, not on
// vmcnt: a wave can look at a word this way while vector loads of its own are
// in flight, where a vector load of the word would only come back after all of
// them (vector loads return in issue order).  Only for words that were stored
// into this XCD's L2 (the XCD-local staging policy).
__device__ __forceinline__ uint64_t ld64_scalar(const uint64_t* p) {
    // The address is the same in every lane; the compiler is told so.
    // (readfirstlane returns int: through uint32_t, or the low half would be
    // sign-extended over the high one.)
    const uint64_t a = (uint64_t)p;
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)a);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
    const uint64_t ua = (uint64_t)lo | ((uint64_t)hi << 32);
    uint64_t v;
    asm volatile("s_load_dwordx2 %0, %1, 0x0 glc\n\ts_waitcnt lgkmcnt(0)"
                 : "=s"(v) : "s"(ua) : "memory");
    return v;
}
// A 32-bit word at agent scope, loaded and waited for inside one asm statement:
// the compiler's count of outstanding vector-memory operations is left as it
// was (it then waits for at most as much as it would have).
__device__ __forceinline__ uint32_t ld32_agent_apart(const void* p) {
    uint32_t v;
    asm volatile("global_load_dword %0, %1, off sc1\n\ts_waitcnt vmcnt(0)"
                 : "=v"(v) : "v"(p) : "memory");
    return v;
}
// Release for data that was stored with scope bits (write-through) or, for the
// XCD-local policy, into the L2 both sides share: once the wave's stores are
// acknowledged they are visible to every load that skips the L1, so waiting
// for them is all a following flag store needs.  (A full agent-scope release,
// buffer_wbl2 sc1, would also write back every unrelated dirty line of the L2
// and measured 15x slower.)
__device__ __forceinline__ void wait_stores_visible() {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// Streaming accesses to the caller's buffers (read once / written once).
__device__ __forceinline__ u32x4 ld128_stream(const void* p) {
    return __builtin_nontemporal_load(as_global(reinterpret_cast<const u32x4*>(p)));
}
__device__ __forceinline__ void st128_stream(void* p, u32x4 v) {
    __builtin_nontemporal_store(v, as_global(reinterpret_cast<u32x4*>(p)));
}
// The same for rows of the caller's buffers in the ring kernels, which may
// start at any byte.
typedef u32x4 u32x4_unaligned __attribute__((aligned(1)));
__device__ __forceinline__ u32x4 ld128_row(const void* p) {
    return __builtin_nontemporal_load((MINT_GLOBAL const u32x4_unaligned*)p);
}
__device__ __forceinline__ void st128_row(void* p, u32x4 v) {
    __builtin_nontemporal_store(v, (MINT_GLOBAL u32x4_unaligned*)p);
}
__device__ __forceinline__ u32x2 ld64_stream(const void* p) {
    return __builtin_nontemporal_load(as_global(reinterpret_cast<const u32x2*>(p)));
}
__device__ __forceinline__ void st64_stream(void* p, u32x2 v) {
    __builtin_nontemporal_store(v, as_global(reinterpret_cast<u32x2*>(p)));
}

// ---- element addition: one IEEE round-to-nearest-even per call ------------
// f16: v_pk_add_f16 (subnormals kept; the kernel is compiled without
// flush-to-zero).  bf16: widen, one binary32 add, round to nearest even
// (v_cvt_pk_bf16_f32), NaN -> 0x7FC0.  f32: v_add_f32.
__device__ __forceinline__ uint32_t add_f16x2(uint32_t a, uint32_t b) {
    f16x2 x = __builtin_bit_cast(f16x2, a), y = __builtin_bit_cast(f16x2, b);
    return __builtin_bit_cast(uint32_t, x + y);
}
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t add_bf16x2(uint32_t a, uint32_t b) {
    f32x2 s;
    s.x = __builtin_bit_cast(float, a << 16) + __builtin_bit_cast(float, b << 16);
    s.y = __builtin_bit_cast(float, a & 0xFFFF0000u) + __builtin_bit_cast(float, b & 0xFFFF0000u);
    // both sums to bf16 in one instruction (v_cvt_pk_bf16_f32: round to nearest
    // even); a NaN becomes the canonical one
    uint32_t bits = __builtin_bit_cast(uint32_t, __builtin_convertvector(s, bf16x2));
    if (s.x != s.x) bits = (bits & 0xFFFF0000u) | 0x7FC0u;
    if (s.y != s.y) bits = (bits & 0x0000FFFFu) | 0x7FC00000u;
    return bits;
}
__device__ __forceinline__ uint32_t add_f32(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t,
                              __builtin_bit_cast(float, a) + __builtin_bit_cast(float, b));
}
template <int DT>
__device__ __forceinline__ uint32_t add_rn(uint32_t a, uint32_t b) {
    if constexpr (DT == DT_F16) return add_f16x2(a, b);
    else if constexpr (DT == DT_BF16) return add_bf16x2(a, b);
    else return add_f32(a, b);
}
template <int DT>
__device__ __forceinline__ u32x4 add_rn(u32x4 a, u32x4 b) {
    u32x4 r;
    r.x = add_rn<DT>(a.x, b.x);
    r.y = add_rn<DT>(a.y, b.y);
    r.z = add_rn<DT>(a.z, b.z);
    r.w = add_rn<DT>(a.w, b.w);
    return r;
}

}  // namespace mint
