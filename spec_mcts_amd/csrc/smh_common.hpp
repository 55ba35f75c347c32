// Shared device helpers for the gfx950 (CDNA4, wave64) kernels of the Q4_0 hot path.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/smh.h"

namespace smh {

typedef _Float16 half_t;
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int WAVE = 64;

// ---- error reporting -------------------------------------------------------------------------
void set_error(const char *fmt, ...);

#define SMH_REQUIRE(cond, ...)            \
    do {                                  \
        if (!(cond)) {                    \
            smh::set_error(__VA_ARGS__);  \
            return -1;                    \
        }                                 \
    } while (0)

inline int launch_status() {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("kernel launch failed: %s", hipGetErrorString(e));
        return (int)e;
    }
    return 0;
}

// ---- bit casts ---------------------------------------------------------------------------------
__device__ __forceinline__ h2 as_h2(uint32_t v) { return __builtin_bit_cast(h2, v); }
__device__ __forceinline__ uint32_t as_u32(h2 v) { return __builtin_bit_cast(uint32_t, v); }

// ---- Q4_0 nibble decoding ------------------------------------------------------------------------
// Codes are two's-complement nibbles in [-8, 7].  XOR with 8 turns a nibble into u = code + 8 in
// [0, 15]; OR-ing u into the mantissa of fp16 1024.0 (0x6400) gives exactly 1024 + u (low nibble)
// or 1024 + 16u (high nibble), from which the code follows with one exact fp16 operation.
constexpr uint32_t NIBBLE_FLIP = 0x88888888u;
constexpr uint32_t MAGIC_1024 = 0x64006400u;

// p holds two offset-binary bytes, one at bits 0-7 and one at bits 16-23.
// Returns the codes of their LOW nibbles as exact fp16 values (.x from bits 0-7, .y from bits 16-23).
__device__ __forceinline__ h2 codes_low(uint32_t p) {
    const h2 off = {(half_t)-1032.0f, (half_t)-1032.0f};
    return as_h2((p & 0x000F000Fu) | MAGIC_1024) + off;
}
// Same for the HIGH nibbles: (1024 + 16u) / 16 - 72 = u - 8, every step exact in fp16.
__device__ __forceinline__ h2 codes_high(uint32_t p) {
    const h2 sixteenth = {(half_t)0.0625f, (half_t)0.0625f};
    const h2 off = {(half_t)-72.0f, (half_t)-72.0f};
    return __builtin_elementwise_fma(as_h2((p & 0x00F000F0u) | MAGIC_1024), sixteenth, off);
}

// Byte `B` of word `even` to bits 0-7 and byte `B` of word `odd` to bits 16-23, other bytes zero.
// v_perm_b32 numbers the bytes of {src0, src1} 0..7 starting at src1's least significant byte;
// selector 0x0c yields 0x00.
template <int B>
__device__ __forceinline__ uint32_t pair_bytes(uint32_t even, uint32_t odd) {
    constexpr uint32_t sel = 0x0c000c00u | (uint32_t)B | ((uint32_t)(4 + B) << 16);
    return __builtin_amdgcn_perm(odd, even, sel);
}
// (lo16 of a, lo16 of b) and (hi16 of a, hi16 of b)
__device__ __forceinline__ uint32_t pack_lo16(uint32_t a, uint32_t b) {
    return __builtin_amdgcn_perm(b, a, 0x05040100u);
}
__device__ __forceinline__ uint32_t pack_hi16(uint32_t a, uint32_t b) {
    return __builtin_amdgcn_perm(b, a, 0x07060302u);
}

// ---- wave reductions -------------------------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
// reductions over the 16 lanes that share lane/16 (one DPP row)
__device__ __forceinline__ float row16_sum(float v) {
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// ---- cross-workgroup hand-off of partial sums ----------------------------------------------------
// Partial results written by one workgroup and read by another (possibly on a different XCD, i.e.
// behind a different L2) travel as device-scope relaxed atomics: such stores write through to the
// point of coherence and such loads never use a possibly stale cache line.  That makes full
// device-scope fences unnecessary (they write back and invalidate the whole L2, which is ruinous
// while other workgroups stream weights through it); all that is needed is that a workgroup's
// stores have completed before its counter increment is issued.
__device__ __forceinline__ void store_coherent(float *p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_coherent(const float *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// wait until every memory operation this wave has issued is complete (stores acknowledged)
__device__ __forceinline__ void wait_memory_ops() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}
// Counts arrivals of the workgroups that share `counter`; returns true in the last one (uniform over
// the workgroup).  Call after store_coherent() of this workgroup's partials; in the last workgroup,
// read the others' partials with load_coherent() and then reset the counter with arrive_reset().
__device__ __forceinline__ bool arrive_is_last(uint32_t *counter, uint32_t expected, uint32_t *s_flag) {
    wait_memory_ops();
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t prev = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *s_flag = (prev == expected - 1u) ? 1u : 0u;
    }
    __syncthreads();
    return *s_flag != 0u;
}
__device__ __forceinline__ void arrive_reset(uint32_t *counter) {
    if (threadIdx.x == 0) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace smh
