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
typedef float f2 __attribute__((ext_vector_type(2)));
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

// The value another lane holds, through a data-parallel-primitive move (no LDS, folds into the instruction that uses it).
// Controls: a permutation of each four consecutive lanes, a rotation of each 16 consecutive lanes (lane i reads i - n), or a
// reversal of each 8 consecutive lanes.
constexpr int DPP_QUAD_XOR1 = 0xB1, DPP_QUAD_XOR2 = 0x4E, DPP_ROW_ROR4 = 0x124, DPP_ROW_ROR8 = 0x128;
constexpr int DPP_ROW_HALF_MIRROR = 0x141;      // lane i of each 8 consecutive lanes reads lane 7 - i
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}

// sum over the 16 lanes that share lane/16 (one DPP row)
__device__ __forceinline__ float row16_sum(float v) {
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// ---- RMSNorm arithmetic shared by every kernel that normalises ---------------------------------------
// Kernels that must agree bit for bit (the RMSNorm launch and the matmul that normalises its own activations) take
// their roundings from here, so that none of them depends on what the compiler chooses to fuse in its context.
__device__ __forceinline__ float sumsq_add(float ss, float x) { return __builtin_fmaf(x, x, ss); }
// fp16(x * r) with the product rounded to fp32 first and to fp16 second, as x.float() * r followed by .half() rounds.
// The empty asm keeps the compiler from merging the two into one mixed-precision multiply that converts on the fly,
// whose results differ from the two roundings in rare last bits.
__device__ __forceinline__ half_t scale_to_half(half_t x, float r) {
    float f = (float)x * r;
    asm("" : "+v"(f));
    return (half_t)f;
}
__device__ __forceinline__ float rms_factor(float total, int n, float eps) {
#pragma clang fp contract(off)
    const float mean = total / (float)n;
    const float shifted = mean + eps;
    return 1.0f / sqrtf(shifted);
}

// ---- cross-workgroup hand-off inside one launch ------------------------------------------------------
// Data written by one workgroup and read by another (possibly on a different XCD, i.e. behind a different
// L2) travels as device-scope relaxed atomics: such stores write through to the point of coherence and
// such loads never use a possibly stale cache line.  Full device-scope fences are avoided (they write back
// and invalidate the whole L2, ruinous while other workgroups stream weights through it); all that is
// needed is that a wave's stores have completed (wait_vmem) before it increments the counter that
// announces them, and that a reader looks at the data only after it has seen the counter.
__device__ __forceinline__ void st_u32(void *p, uint32_t v) {
    __hip_atomic_store(reinterpret_cast<uint32_t *>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t ld_u32(const void *p) {
    return __hip_atomic_load(reinterpret_cast<const uint32_t *>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_u64(void *p, u32x2 v) {
    __hip_atomic_store(reinterpret_cast<uint64_t *>(p), __builtin_bit_cast(uint64_t, v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ u32x2 ld_u64(const void *p) {
    return __builtin_bit_cast(u32x2, __hip_atomic_load(reinterpret_cast<const uint64_t *>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}
__device__ __forceinline__ void st_f32(float *p, float v) { st_u32(p, __builtin_bit_cast(uint32_t, v)); }
__device__ __forceinline__ float ld_f32(const float *p) { return __builtin_bit_cast(float, ld_u32(p)); }
// (whole-vector bit casts only: __builtin_bit_cast applied to ONE ELEMENT of an ext_vector reads element 0)
__device__ __forceinline__ void st_f4(float *p, f4 v) {
    const u32x4 u = __builtin_bit_cast(u32x4, v);
    st_u64(p, u32x2{u[0], u[1]});
    st_u64(p + 2, u32x2{u[2], u[3]});
}
__device__ __forceinline__ f4 ld_f4(const float *p) {
    const u32x2 a = ld_u64(p), b = ld_u64(p + 2);
    return __builtin_bit_cast(f4, u32x4{a[0], a[1], b[0], b[1]});
}
__device__ __forceinline__ h4 ld_h4(const half_t *p) { return __builtin_bit_cast(h4, ld_u64(p)); }
__device__ __forceinline__ void st_h4(half_t *p, h4 v) { st_u64(p, __builtin_bit_cast(u32x2, v)); }
__device__ __forceinline__ void wait_vmem() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

}  // namespace smh
