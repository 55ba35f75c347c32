// Flat Q4_0 codec kernels: 64-byte rows of packed signed nibbles <-> fp16.
//
// Both kernels are pure streaming (HBM-bound): dequant reads 68 B and writes 256 B per row,
// quantise reads 256 B and writes 68 B per row.  One lane owns 16 bytes of a row, so a row is
// covered by 4 neighbouring lanes and every access is a 128-bit load/store.
#include "q40_matmul.hpp"

namespace smh {

// out[row*128 + j]      = code(high nibble of byte j) * s[2*row]
// out[row*128 + 64 + j] = code(low  nibble of byte j) * s[2*row+1]      (one fp16 multiply each)
__global__ __launch_bounds__(256) void q40_dequant_kernel(const u32x4 *__restrict__ w,
                                                          const uint32_t *__restrict__ s,
                                                          half_t *__restrict__ out, long rows) {
    long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
    long row = t >> 2;
    int c = (int)(t & 3);
    if (row >= rows) return;
    u32x4 v = w[row * 4 + c];
    uint32_t sp = s[row];                       // (s[2row], s[2row+1])
    h2 s_hi = as_h2(pack_lo16(sp, sp));
    h2 s_lo = as_h2(pack_hi16(sp, sp));
    uint32_t hi[8], lo[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        uint32_t u = v[j] ^ NIBBLE_FLIP;
        uint32_t u1 = u >> 8;
        // pairs (byte0, byte2) and (byte1, byte3) of this word
        uint32_t h02 = as_u32(codes_high(u) * s_hi), h13 = as_u32(codes_high(u1) * s_hi);
        uint32_t l02 = as_u32(codes_low(u) * s_lo), l13 = as_u32(codes_low(u1) * s_lo);
        hi[2 * j] = pack_lo16(h02, h13);        // (byte0, byte1)
        hi[2 * j + 1] = pack_hi16(h02, h13);    // (byte2, byte3)
        lo[2 * j] = pack_lo16(l02, l13);
        lo[2 * j + 1] = pack_hi16(l02, l13);
    }
    u32x4 *o_hi = reinterpret_cast<u32x4 *>(out + row * 128 + c * 16);
    u32x4 *o_lo = reinterpret_cast<u32x4 *>(out + row * 128 + 64 + c * 16);
    o_hi[0] = u32x4{hi[0], hi[1], hi[2], hi[3]};
    o_hi[1] = u32x4{hi[4], hi[5], hi[6], hi[7]};
    o_lo[0] = u32x4{lo[0], lo[1], lo[2], lo[3]};
    o_lo[1] = u32x4{lo[4], lo[5], lo[6], lo[7]};
}

// One fp16 value -> code with torch's semantics: q = fp16(x / scale); code = rint(q) (to nearest
// even); NaN (0/0) -> 0.  The division is a correctly rounded fp32 division rounded once more to fp16.
__device__ __forceinline__ int q40_code(half_t x, float scale) {
    half_t q = (half_t)((float)x / scale);
    float qf = (float)q;
    if (!(qf == qf)) return 0;
    return (int)__builtin_rintf(qf);
}

// Lane layout: 8 lanes per 64-value group (8 values = one 128-bit load each), so a wave covers
// 8 groups = 4 packed rows.  absmax is reduced over the 8 lanes of a group with xor-shuffles.
__global__ __launch_bounds__(256) void q40_quantize_kernel(const u32x4 *__restrict__ in,
                                                           uint8_t *__restrict__ w,
                                                           half_t *__restrict__ s, long groups) {
    long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
    long g = t >> 3;
    int c = (int)(t & 7);
    bool live = g < groups;
    u32x4 raw = live ? in[t] : u32x4{0, 0, 0, 0};
    half_t x[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        h2 p = as_h2(raw[j]);
        x[2 * j] = p.x;
        x[2 * j + 1] = p.y;
    }
    // |x| as bit patterns: for finite values the integer order is the magnitude order
    uint32_t amax = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        uint32_t a = raw[j] & 0x7FFF7FFFu;
        uint32_t m = max(a & 0xFFFFu, a >> 16);
        amax = max(amax, m);
    }
#pragma unroll
    for (int o = 4; o > 0; o >>= 1) amax = max(amax, (uint32_t)__shfl_xor((int)amax, o, 64));
    half_t amax_h = __builtin_bit_cast(half_t, (uint16_t)amax);
    half_t scale_h = (half_t)((float)amax_h / 7.0f);
    float scale = (float)scale_h;
    uint32_t nib = 0;   // 8 codes, value j in bits 4j..4j+3
#pragma unroll
    for (int j = 0; j < 8; ++j) nib |= (uint32_t)(q40_code(x[j], scale) & 15) << (4 * j);
    // the partner group (g ^ 1) sits 8 lanes away; even groups supply high nibbles
    uint32_t other = (uint32_t)__shfl_xor((int)nib, 8, 64);
    if (!live) return;
    if (c == 0) s[g] = scale_h;
    if ((g & 1) == 0) {
        uint32_t hi = nib, lo = other;
        uint32_t b0 = 0, b1 = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            b0 |= ((((hi >> (4 * j)) & 15) << 4) | ((lo >> (4 * j)) & 15)) << (8 * j);
            b1 |= ((((hi >> (4 * j + 16)) & 15) << 4) | ((lo >> (4 * j + 16)) & 15)) << (8 * j);
        }
        u32x2 *dst = reinterpret_cast<u32x2 *>(w + (g >> 1) * 64 + c * 8);
        *dst = u32x2{b0, b1};
    }
}

// The same quantiser for checkpoint weights held in fp32 or bfloat16 (passed widened to fp32, which is exact).  torch's
// arithmetic for those types (fp16_to_int4.py:60-70 run on such a tensor): wmax / 7.0 is rounded to the tensor's own
// type (fp32, or bfloat16) and then to fp16; w / scale promotes to fp32, so the quotient is NOT rounded to fp16 before
// round-half-even; 0 / 0 -> NaN -> code 0.  SRC_BF16 selects the intermediate bfloat16 rounding of the scale.
__device__ __forceinline__ float round_to_bf16(float x) {
    uint32_t u = __builtin_bit_cast(uint32_t, x);
    if ((u & 0x7F800000u) == 0x7F800000u) return x;                  // inf / nan stay
    u += 0x7FFFu + ((u >> 16) & 1u);
    return __builtin_bit_cast(float, u & 0xFFFF0000u);
}
template <bool SRC_BF16>
__global__ __launch_bounds__(256) void q40_quantize_f32_kernel(const f4 *__restrict__ in, uint8_t *__restrict__ w,
                                                               half_t *__restrict__ s, long groups) {
    long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
    long g = t >> 3;
    int c = (int)(t & 7);
    bool live = g < groups;
    f4 a = live ? in[2 * t] : f4{0.f, 0.f, 0.f, 0.f}, b = live ? in[2 * t + 1] : f4{0.f, 0.f, 0.f, 0.f};
    const float x[8] = {a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]};
    float amax = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(x[j]));
#pragma unroll
    for (int o = 4; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
    float q7 = amax / 7.0f;
    if (SRC_BF16) q7 = round_to_bf16(q7);
    const half_t scale_h = (half_t)q7;
    const float scale = (float)scale_h;
    uint32_t nib = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float qf = x[j] / scale;
        const int code = (qf == qf) ? (int)__builtin_rintf(qf) : 0;
        nib |= (uint32_t)(code & 15) << (4 * j);
    }
    uint32_t other = (uint32_t)__shfl_xor((int)nib, 8, 64);
    if (!live) return;
    if (c == 0) s[g] = scale_h;
    if ((g & 1) == 0) {
        uint32_t hi = nib, lo = other;
        uint32_t b0 = 0, b1 = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            b0 |= ((((hi >> (4 * j)) & 15) << 4) | ((lo >> (4 * j)) & 15)) << (8 * j);
            b1 |= ((((hi >> (4 * j + 16)) & 15) << 4) | ((lo >> (4 * j + 16)) & 15)) << (8 * j);
        }
        *reinterpret_cast<u32x2 *>(w + (g >> 1) * 64 + c * 8) = u32x2{b0, b1};
    }
}

// One thread per output dword of the tiled layout (q40_matmul.hpp): 1024 nibble dwords + 64 scale dwords per tile.
__global__ __launch_bounds__(256) void q40_tile_kernel(const uint8_t *__restrict__ w, const half_t *__restrict__ s,
                                                       int K, int N, uint32_t *__restrict__ tiled, long tiles) {
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    constexpr int DW = TILE_BYTES / 4;
    if (idx >= tiles * DW) return;
    const long tile = idx / DW;
    const int d = (int)(idx - tile * DW);
    const long steps = tiled_steps(K);
    const int unit = (int)(tile / steps), step = (int)(tile - (long)unit * steps);
    uint32_t out;
    if (d < TILE_W_BYTES / 4) {
        const int q = d >> 8, lane = (d >> 2) & 63, e = d & 3;         // piece, lane, dword of the lane's 16 bytes
        const int g = lane >> 4, c = lane & 15, blk = q >> 1, B = 2 * (q & 1) + (e >> 1);
        const long col = (long)unit * 128 + 64 * blk + 4 * c + B;       // byte column of the checkpoint row
        const int r0 = 32 * step + 8 * g + ((e & 1) ? 2 : 0);           // x: rows 0,4,1,5; x2: rows 2,6,3,7
        const int rows[4] = {r0, r0 + 4, r0 + 1, r0 + 5};
        out = 0;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            uint32_t byte = 0;                                           // code 0 | code 0 before the flip
            if (rows[b] < K && col < N / 2) byte = w[(long)rows[b] * (N / 2) + col];
            out |= (byte ^ 0x88u) << (8 * b);
        }
    } else {
        const int e = d - TILE_W_BYTES / 4;                              // [g][group][i / 2]
        const int g = e >> 4, grp = (e >> 2) & 3, i = 2 * (e & 3);
        const long gcol = (long)unit * 4 + grp;
        uint32_t v[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int row = 32 * step + 8 * g + i + h;
            v[h] = (row < K && gcol < N / 64) ? __builtin_bit_cast(uint16_t, s[(long)row * (N / 64) + gcol]) : 0u;
        }
        out = v[0] | (v[1] << 16);
    }
    tiled[idx] = out;
}

}  // namespace smh

extern "C" size_t smh_q40_tiled_bytes(int K, int N) {
    if (K <= 0 || N <= 0) return 0;
    return (size_t)smh::tiled_units(N) * smh::tiled_steps(K) * smh::TILE_BYTES;
}

extern "C" int smh_q40_tile(const void *w, const void *s, int K, int N, void *tiled, size_t tiled_bytes, smh_stream_t stream) {
    using namespace smh;
    SMH_REQUIRE(K > 0 && N > 0 && N % 128 == 0, "smh_q40_tile: K=%d N=%d (N must be a positive multiple of 128)", K, N);
    SMH_REQUIRE(w && s && tiled, "smh_q40_tile: null pointer");
    SMH_REQUIRE(tiled_bytes >= smh_q40_tiled_bytes(K, N), "smh_q40_tile: buffer %zu < %zu bytes", tiled_bytes, smh_q40_tiled_bytes(K, N));
    SMH_REQUIRE(((uintptr_t)tiled & 127) == 0, "smh_q40_tile: the tiled buffer must be 128-byte aligned");
    const long tiles = tiled_units(N) * tiled_steps(K);
    const long threads = tiles * (TILE_BYTES / 4);
    hipLaunchKernelGGL(q40_tile_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint8_t *)w, (const half_t *)s, K, N, (uint32_t *)tiled, tiles);
    return launch_status();
}

extern "C" int smh_q40_dequant(const void *w, const void *s, void *out, long rows, smh_stream_t stream) {
    using namespace smh;
    SMH_REQUIRE(rows >= 0, "smh_q40_dequant: rows=%ld", rows);
    if (rows == 0) return 0;
    SMH_REQUIRE(w && s && out, "smh_q40_dequant: null pointer");
    long threads = rows * 4;
    dim3 grid((unsigned)((threads + 255) / 256));
    hipLaunchKernelGGL(q40_dequant_kernel, grid, dim3(256), 0, (hipStream_t)stream,
                       (const u32x4 *)w, (const uint32_t *)s, (half_t *)out, rows);
    return launch_status();
}

// ---- the block-of-32 flavour (scale = absmax / 8, codes 0..15 with offset 8, elements j and j + 16 share byte j) ----
// one thread per block: 16 bytes + one fp16 scale <-> 32 fp16 values
namespace smh {
__global__ __launch_bounds__(256) void gq40_dequant_kernel(const u32x4 *__restrict__ packed, const half_t *__restrict__ scale,
                                                           half_t *__restrict__ out, long blocks) {
    const long b = (long)blockIdx.x * 256 + threadIdx.x;
    if (b >= blocks) return;
    const u32x4 v = packed[b];
    const half_t sc = scale[b];
    half_t lo[16], hi[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const uint32_t byte = (v[j >> 2] >> (8 * (j & 3))) & 255u;
        lo[j] = (half_t)(float)((int)(byte & 15u) - 8) * sc;         // exact small integer times the scale: one fp16 rounding
        hi[j] = (half_t)(float)((int)(byte >> 4) - 8) * sc;
    }
    u32x4 *o = reinterpret_cast<u32x4 *>(out + b * 32);
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        o[q] = u32x4{as_u32(h2{lo[8 * q], lo[8 * q + 1]}), as_u32(h2{lo[8 * q + 2], lo[8 * q + 3]}),
                     as_u32(h2{lo[8 * q + 4], lo[8 * q + 5]}), as_u32(h2{lo[8 * q + 6], lo[8 * q + 7]})};
        o[2 + q] = u32x4{as_u32(h2{hi[8 * q], hi[8 * q + 1]}), as_u32(h2{hi[8 * q + 2], hi[8 * q + 3]}),
                         as_u32(h2{hi[8 * q + 4], hi[8 * q + 5]}), as_u32(h2{hi[8 * q + 6], hi[8 * q + 7]})};
    }
}

// rint(fp16(x / scale)) cut to -8 .. 8 while still a float (a scale that underflowed to 0 gives +-inf), NaN (0 / 0) -> 0
__device__ __forceinline__ int gq40_code(half_t x, float scale) {
    const float qf = (float)(half_t)((float)x / scale);
    if (!(qf == qf)) return 0;
    return (int)__builtin_rintf(fminf(fmaxf(qf, -8.0f), 8.0f));
}

__global__ __launch_bounds__(256) void gq40_quantize_kernel(const u32x4 *__restrict__ in, u32x4 *__restrict__ packed,
                                                            half_t *__restrict__ scale, long blocks) {
    const long b = (long)blockIdx.x * 256 + threadIdx.x;
    if (b >= blocks) return;
    half_t x[32];
    uint32_t amax = 0;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const u32x4 r = in[b * 4 + q];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const h2 pr = as_h2(r[j]);
            x[8 * q + 2 * j] = pr.x;
            x[8 * q + 2 * j + 1] = pr.y;
            const uint32_t a = r[j] & 0x7FFF7FFFu;                  // |x| as bit patterns: integer order = magnitude order
            amax = max(amax, max(a & 0xFFFFu, a >> 16));
        }
    }
    const half_t scale_h = (half_t)((float)__builtin_bit_cast(half_t, (uint16_t)amax) / 8.0f);
    const float sf = (float)scale_h;
    uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const int ql = min(gq40_code(x[j], sf) + 8, 15), qh = min(gq40_code(x[j + 16], sf) + 8, 15);
        w[j >> 2] |= (uint32_t)(ql | (qh << 4)) << (8 * (j & 3));
    }
    packed[b] = u32x4{w[0], w[1], w[2], w[3]};
    scale[b] = scale_h;
}
}  // namespace smh

extern "C" int smh_gq40_dequant(const void *packed, const void *scale, void *out, long blocks, smh_stream_t stream) {
    using namespace smh;
    SMH_REQUIRE(blocks >= 0, "smh_gq40_dequant: blocks=%ld", blocks);
    if (blocks == 0) return 0;
    SMH_REQUIRE(packed && scale && out && (((uintptr_t)packed | (uintptr_t)out) & 15) == 0, "smh_gq40_dequant: null or misaligned pointer");
    hipLaunchKernelGGL(gq40_dequant_kernel, dim3((unsigned)((blocks + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const u32x4 *)packed, (const half_t *)scale, (half_t *)out, blocks);
    return launch_status();
}

extern "C" int smh_gq40_quantize(const void *in, void *packed, void *scale, long blocks, smh_stream_t stream) {
    using namespace smh;
    SMH_REQUIRE(blocks >= 0, "smh_gq40_quantize: blocks=%ld", blocks);
    if (blocks == 0) return 0;
    SMH_REQUIRE(in && packed && scale && (((uintptr_t)in | (uintptr_t)packed) & 15) == 0, "smh_gq40_quantize: null or misaligned pointer");
    hipLaunchKernelGGL(gq40_quantize_kernel, dim3((unsigned)((blocks + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const u32x4 *)in, (u32x4 *)packed, (half_t *)scale, blocks);
    return launch_status();
}

extern "C" int smh_q40_quantize(const void *in, void *w, void *s, long groups, smh_stream_t stream) {
    using namespace smh;
    SMH_REQUIRE(groups >= 0 && (groups & 1) == 0, "smh_q40_quantize: groups=%ld must be even", groups);
    if (groups == 0) return 0;
    SMH_REQUIRE(in && w && s, "smh_q40_quantize: null pointer");
    long threads = groups * 8;
    dim3 grid((unsigned)((threads + 255) / 256));
    hipLaunchKernelGGL(q40_quantize_kernel, grid, dim3(256), 0, (hipStream_t)stream,
                       (const u32x4 *)in, (uint8_t *)w, (half_t *)s, groups);
    return launch_status();
}

extern "C" int smh_q40_quantize_f32(const void *in, int src_bf16, void *w, void *s, long groups, smh_stream_t stream) {
    using namespace smh;
    SMH_REQUIRE(groups >= 0 && (groups & 1) == 0, "smh_q40_quantize_f32: groups=%ld must be even", groups);
    if (groups == 0) return 0;
    SMH_REQUIRE(in && w && s && ((uintptr_t)in & 15) == 0, "smh_q40_quantize_f32: null or misaligned pointer");
    long threads = groups * 8;
    dim3 grid((unsigned)((threads + 255) / 256));
    if (src_bf16) hipLaunchKernelGGL(q40_quantize_f32_kernel<true>, grid, dim3(256), 0, (hipStream_t)stream, (const f4 *)in, (uint8_t *)w, (half_t *)s, groups);
    else hipLaunchKernelGGL(q40_quantize_f32_kernel<false>, grid, dim3(256), 0, (hipStream_t)stream, (const f4 *)in, (uint8_t *)w, (half_t *)s, groups);
    return launch_status();
}
