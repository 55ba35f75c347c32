// RoPE on a (d, d + 64) pair and the Q4_0 append of one 128-wide K or V row, as one wave (lane = d).
#pragma once

#include "smh_common.hpp"

namespace smh {

// ---- RoPE + Q4_0 KV append from the fused q|k|v product ------------------------------------------------
__device__ __forceinline__ void rope_pair2(half_t &x1, half_t &x2, half_t cs, half_t sn) {
#pragma clang fp contract(off)      // the two products are rounded to fp16 before they are added
    half_t a = x1 * cs, b = (-x2) * sn;
    half_t c = x2 * cs, d = x1 * sn;
    x1 = a + b;
    x2 = c + d;
}
__device__ __forceinline__ int kv_code2(half_t x, float scale) {
    float qf = (float)(half_t)((float)x / scale);
    if (!(qf == qf)) return 0;
    return (int)__builtin_rintf(qf);
}
__device__ __forceinline__ void kv_store_row2(half_t lo, half_t hi, uint8_t *row, half_t *scales, int lane) {
    uint32_t a_lo = (uint32_t)(__builtin_bit_cast(uint16_t, lo) & 0x7FFFu);
    uint32_t a_hi = (uint32_t)(__builtin_bit_cast(uint16_t, hi) & 0x7FFFu);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        a_lo = max(a_lo, (uint32_t)__shfl_xor((int)a_lo, o, 64));
        a_hi = max(a_hi, (uint32_t)__shfl_xor((int)a_hi, o, 64));
    }
    half_t s0 = (half_t)((float)__builtin_bit_cast(half_t, (uint16_t)a_lo) / 7.0f);
    half_t s1 = (half_t)((float)__builtin_bit_cast(half_t, (uint16_t)a_hi) / 7.0f);
    int c0 = kv_code2(lo, (float)s0), c1 = kv_code2(hi, (float)s1);
    row[lane] = (uint8_t)(((c0 & 15) << 4) | (c1 & 15));
    if (lane == 0) { scales[0] = s0; scales[1] = s1; }
}

}  // namespace smh
