// Small fused kernels around the Q4_0 linears: RMSNorm, SiLU*up, greedy argmax, RoPE (+ Q4_0
// append of the new K/V row) and the branch fork copy.  All are launch- or HBM-bound; the point of
// fusing is to keep a decode step at a handful of launches, not arithmetic.
#include "smh_common.hpp"

namespace smh {

// ---- RMSNorm: fp32 normalise -> fp16 -> * weight -> fp16 ------------------------------------------
// one workgroup per row; dim % 8 == 0
__global__ __launch_bounds__(256) void rmsnorm_kernel(const half_t *__restrict__ x, const half_t *__restrict__ wt,
                                                      half_t *__restrict__ out, int dim, float eps) {
    __shared__ float s_part[4];
    const long row = blockIdx.x;
    const half_t *xr = x + row * dim;
    half_t *orow = out + row * dim;
    float ss = 0.f;
    for (int i = threadIdx.x * 8; i < dim; i += 256 * 8) {
        h8 v = *reinterpret_cast<const h8 *>(xr + i);
#pragma unroll
        for (int j = 0; j < 8; ++j) ss += (float)v[j] * (float)v[j];
    }
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float total = s_part[0] + s_part[1] + s_part[2] + s_part[3];
    const float r = 1.0f / sqrtf(total / (float)dim + eps);
    for (int i = threadIdx.x * 8; i < dim; i += 256 * 8) {
        h8 v = *reinterpret_cast<const h8 *>(xr + i);
        h8 w = *reinterpret_cast<const h8 *>(wt + i);
        h8 o;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            half_t n = (half_t)((float)v[j] * r);
            o[j] = n * w[j];
        }
        *reinterpret_cast<h8 *>(orow + i) = o;
    }
}

// ---- SwiGLU gate: fp16(silu(g)) * u ------------------------------------------------------------------
__global__ __launch_bounds__(256) void silu_mul_kernel(const half_t *__restrict__ g, const half_t *__restrict__ u,
                                                       half_t *__restrict__ out, long n) {
    long i = ((long)blockIdx.x * 256 + threadIdx.x) * 8;
    if (i + 8 <= n) {
        h8 a = *reinterpret_cast<const h8 *>(g + i);
        h8 b = *reinterpret_cast<const h8 *>(u + i);
        h8 o;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            float af = (float)a[j];
            half_t sl = (half_t)(af / (1.0f + expf(-af)));
            o[j] = sl * b[j];
        }
        *reinterpret_cast<h8 *>(out + i) = o;
    } else {
        for (; i < n; ++i) {
            float af = (float)g[i];
            half_t sl = (half_t)(af / (1.0f + expf(-af)));
            out[i] = sl * u[i];
        }
    }
}

// ---- greedy pick: largest logit, lowest index on ties --------------------------------------------------
__device__ __forceinline__ void argmax_merge(float &bv, int &bi, float v, int i) {
    if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
}
// one workgroup of 1024 threads per row; 128-bit loads, four in flight per thread, when the row allows them
__global__ __launch_bounds__(1024) void argmax_kernel(const half_t *__restrict__ logits, int vocab, long ld,
                                                      int64_t *__restrict__ out) {
    __shared__ float s_v[16];
    __shared__ int s_i[16];
    const half_t *row = logits + (long)blockIdx.x * ld;
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    const bool wide = (ld % 8 == 0) && ((reinterpret_cast<uintptr_t>(logits) & 15) == 0);
    const int chunks = wide ? vocab / 8 : 0;
    for (int c0 = threadIdx.x; c0 < chunks; c0 += 4 * 1024) {
        h8 v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = c0 + 1024 * j;
            if (c < chunks) v[j] = *reinterpret_cast<const h8 *>(row + 8 * c);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = c0 + 1024 * j;
            if (c < chunks) {
#pragma unroll
                for (int e = 0; e < 8; ++e) argmax_merge(bv, bi, (float)v[j][e], 8 * c + e);
            }
        }
    }
    for (int i = 8 * chunks + threadIdx.x; i < vocab; i += 1024) argmax_merge(bv, bi, (float)row[i], i);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        float ov = __shfl_xor(bv, o, 64);
        int oi = __shfl_xor(bi, o, 64);
        argmax_merge(bv, bi, ov, oi);
    }
    if ((threadIdx.x & 63) == 0) { s_v[threadIdx.x >> 6] = bv; s_i[threadIdx.x >> 6] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 16; ++w) argmax_merge(bv, bi, s_v[w], s_i[w]);
        out[blockIdx.x] = (bi == 0x7fffffff) ? 0 : bi;
    }
}

// ---- RoPE, rotate-half form, three fp16 roundings per element ----------------------------------------
// lane i of a wave owns the pair (i, i + 64) of one 128-wide head vector
__device__ __forceinline__ void rope_pair(half_t &x1, half_t &x2, half_t cs, half_t sn) {
#pragma clang fp contract(off)      // the two products are rounded to fp16 before they are added
    half_t a = x1 * cs, b = (-x2) * sn;     // q*cos, rotate_half(q)*sin for the first half
    half_t c = x2 * cs, d = x1 * sn;        // same for the second half
    x1 = a + b;
    x2 = c + d;
}

// code = rint(fp16(x / scale)), NaN -> 0 (same as the flat quantiser)
__device__ __forceinline__ int kv_code(half_t x, float scale) {
    float qf = (float)(half_t)((float)x / scale);
    if (!(qf == qf)) return 0;
    return (int)__builtin_rintf(qf);
}

// Quantise one 128-wide vector held as (lo = element lane, hi = element lane+64) into one packed row.
__device__ __forceinline__ void kv_store_row(half_t lo, half_t hi, uint8_t *row, half_t *scales, int lane) {
    uint32_t a_lo = (uint32_t)(__builtin_bit_cast(uint16_t, lo) & 0x7FFFu);
    uint32_t a_hi = (uint32_t)(__builtin_bit_cast(uint16_t, hi) & 0x7FFFu);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        a_lo = max(a_lo, (uint32_t)__shfl_xor((int)a_lo, o, 64));
        a_hi = max(a_hi, (uint32_t)__shfl_xor((int)a_hi, o, 64));
    }
    half_t s0 = (half_t)((float)__builtin_bit_cast(half_t, (uint16_t)a_lo) / 7.0f);   // group of elements 0..63
    half_t s1 = (half_t)((float)__builtin_bit_cast(half_t, (uint16_t)a_hi) / 7.0f);   // group of elements 64..127
    int c0 = kv_code(lo, (float)s0), c1 = kv_code(hi, (float)s1);
    row[lane] = (uint8_t)(((c0 & 15) << 4) | (c1 & 15));
    if (lane == 0) { scales[0] = s0; scales[1] = s1; }
}

// decode step: one wave per (branch, head); heads 0..H-1 are queries, H..H+Hkv-1 are key/value heads
__global__ __launch_bounds__(256) void rope_append_kv_kernel(half_t *__restrict__ q, half_t *__restrict__ k,
                                                             const half_t *__restrict__ v, int B, int H, int Hkv,
                                                             const half_t *__restrict__ cos_tab, const half_t *__restrict__ sin_tab,
                                                             const int32_t *__restrict__ pos_dev,
                                                             uint8_t *__restrict__ cache_k, half_t *__restrict__ cache_ks,
                                                             uint8_t *__restrict__ cache_v, half_t *__restrict__ cache_vs,
                                                             int Smax, const int32_t *__restrict__ t_dev) {
    const int lane = threadIdx.x & 63;
    const long item = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int heads = H + Hkv;
    if (item >= (long)B * heads) return;
    const int b = (int)(item / heads);
    const int h = (int)(item % heads);
    const int pos = *pos_dev;
    const half_t cs = cos_tab[(long)pos * 64 + lane];
    const half_t sn = sin_tab[(long)pos * 64 + lane];
    if (h < H) {
        half_t *p = q + ((long)b * H + h) * 128;
        half_t x1 = p[lane], x2 = p[lane + 64];
        rope_pair(x1, x2, cs, sn);
        p[lane] = x1;
        p[lane + 64] = x2;
        return;
    }
    const int hk = h - H;
    half_t *pk = k + ((long)b * Hkv + hk) * 128;
    half_t x1 = pk[lane], x2 = pk[lane + 64];
    rope_pair(x1, x2, cs, sn);
    pk[lane] = x1;
    pk[lane + 64] = x2;
    if (cache_k == nullptr) return;
    const int t = *t_dev;
    if (t < 0 || t >= Smax) return;
    const long row = ((long)b * Smax + t) * Hkv + hk;
    kv_store_row(x1, x2, cache_k + row * 64, cache_ks + row * 2, lane);
    const half_t *pv = v + ((long)b * Hkv + hk) * 128;
    kv_store_row(pv[lane], pv[lane + 64], cache_v + row * 64, cache_vs + row * 2, lane);
}

// prefill: q [S,H,128], k [S,Hkv,128]; token s sits at position pos0 + s
__global__ __launch_bounds__(256) void rope_kernel(half_t *__restrict__ q, half_t *__restrict__ k, int S, int H, int Hkv,
                                                   const half_t *__restrict__ cos_tab, const half_t *__restrict__ sin_tab, int pos0) {
    const int lane = threadIdx.x & 63;
    const long item = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int heads = H + Hkv;
    if (item >= (long)S * heads) return;
    const int s = (int)(item / heads);
    const int h = (int)(item % heads);
    const half_t cs = cos_tab[(long)(pos0 + s) * 64 + lane];
    const half_t sn = sin_tab[(long)(pos0 + s) * 64 + lane];
    half_t *p = (h < H) ? q + ((long)s * H + h) * 128 : k + ((long)s * Hkv + (h - H)) * 128;
    half_t x1 = p[lane], x2 = p[lane + 64];
    rope_pair(x1, x2, cs, sn);
    p[lane] = x1;
    p[lane + 64] = x2;
}

// ---- fork: copy one branch's cache row to `forks` other branches ------------------------------------------
__global__ __launch_bounds__(256) void kv_fork_kernel(u32x4 *__restrict__ cache, long row_vec, int origin, int curr) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= row_vec) return;
    const int dst = curr + blockIdx.y;
    cache[(long)dst * row_vec + i] = cache[(long)origin * row_vec + i];
}

}  // namespace smh

extern "C" int smh_rmsnorm(const void *x, const void *weight, void *out, int rows, int dim, float eps, smh_stream_t stream) {
    using namespace smh;
    SMH_REQUIRE(rows >= 0 && dim > 0 && dim % 8 == 0, "smh_rmsnorm: rows=%d dim=%d (dim must be a multiple of 8)", rows, dim);
    if (rows == 0) return 0;
    SMH_REQUIRE(x && weight && out, "smh_rmsnorm: null pointer");
    hipLaunchKernelGGL(rmsnorm_kernel, dim3(rows), dim3(256), 0, (hipStream_t)stream,
                       (const half_t *)x, (const half_t *)weight, (half_t *)out, dim, eps);
    return launch_status();
}

extern "C" int smh_silu_mul(const void *g, const void *u, void *out, long n, smh_stream_t stream) {
    using namespace smh;
    SMH_REQUIRE(n >= 0, "smh_silu_mul: n=%ld", n);
    if (n == 0) return 0;
    SMH_REQUIRE(g && u && out, "smh_silu_mul: null pointer");
    long blocks = (n + 2047) / 2048;
    hipLaunchKernelGGL(silu_mul_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const half_t *)g, (const half_t *)u, (half_t *)out, n);
    return launch_status();
}

extern "C" int smh_argmax(const void *logits, int rows, int vocab, long ld, int64_t *out, smh_stream_t stream) {
    using namespace smh;
    SMH_REQUIRE(rows >= 0 && vocab > 0 && ld >= vocab, "smh_argmax: rows=%d vocab=%d ld=%ld", rows, vocab, ld);
    if (rows == 0) return 0;
    SMH_REQUIRE(logits && out, "smh_argmax: null pointer");
    hipLaunchKernelGGL(argmax_kernel, dim3(rows), dim3(1024), 0, (hipStream_t)stream, (const half_t *)logits, vocab, ld, out);
    return launch_status();
}

extern "C" int smh_rope_append_kv(void *q, void *k, const void *v, int B, int H, int Hkv, int D,
                                  const void *cos_tab, const void *sin_tab, const int32_t *pos_dev,
                                  void *cache_k, void *cache_ks, void *cache_v, void *cache_vs,
                                  int Smax, const int32_t *t_dev, smh_stream_t stream) {
    using namespace smh;
    SMH_REQUIRE(D == 128, "smh_rope_append_kv: head dim %d (only 128)", D);
    SMH_REQUIRE(B >= 0 && H > 0 && Hkv > 0, "smh_rope_append_kv: B=%d H=%d Hkv=%d", B, H, Hkv);
    if (B == 0) return 0;
    SMH_REQUIRE(q && k && cos_tab && sin_tab && pos_dev, "smh_rope_append_kv: null pointer");
    SMH_REQUIRE(!cache_k || (v && cache_ks && cache_v && cache_vs && t_dev && Smax > 0), "smh_rope_append_kv: cache arguments incomplete");
    long items = (long)B * (H + Hkv);
    hipLaunchKernelGGL(rope_append_kv_kernel, dim3((unsigned)((items + 3) / 4)), dim3(256), 0, (hipStream_t)stream,
                       (half_t *)q, (half_t *)k, (const half_t *)v, B, H, Hkv, (const half_t *)cos_tab, (const half_t *)sin_tab,
                       pos_dev, (uint8_t *)cache_k, (half_t *)cache_ks, (uint8_t *)cache_v, (half_t *)cache_vs, Smax, t_dev);
    return launch_status();
}

extern "C" int smh_rope(void *q, void *k, int S, int H, int Hkv, int D, const void *cos_tab, const void *sin_tab,
                        int pos0, smh_stream_t stream) {
    using namespace smh;
    SMH_REQUIRE(D == 128, "smh_rope: head dim %d (only 128)", D);
    SMH_REQUIRE(S >= 0 && H > 0 && Hkv > 0 && pos0 >= 0, "smh_rope: S=%d H=%d Hkv=%d pos0=%d", S, H, Hkv, pos0);
    if (S == 0) return 0;
    SMH_REQUIRE(q && k && cos_tab && sin_tab, "smh_rope: null pointer");
    long items = (long)S * (H + Hkv);
    hipLaunchKernelGGL(rope_kernel, dim3((unsigned)((items + 3) / 4)), dim3(256), 0, (hipStream_t)stream,
                       (half_t *)q, (half_t *)k, S, H, Hkv, (const half_t *)cos_tab, (const half_t *)sin_tab, pos0);
    return launch_status();
}

extern "C" int smh_kv_fork(void *cache, void *cache_s, int Bmax, long row_bytes, long row_scales,
                           int origin, int curr, int forks, smh_stream_t stream) {
    using namespace smh;
    SMH_REQUIRE(forks >= 0 && origin >= 0 && origin < Bmax && curr >= 0 && curr + forks <= Bmax,
                "smh_kv_fork: origin=%d curr=%d forks=%d Bmax=%d", origin, curr, forks, Bmax);
    SMH_REQUIRE(origin < curr || origin >= curr + forks, "smh_kv_fork: origin inside the destination range");
    SMH_REQUIRE(row_bytes % 16 == 0 && (row_scales * 2) % 16 == 0, "smh_kv_fork: rows must be multiples of 16 bytes");
    if (forks == 0) return 0;
    SMH_REQUIRE(cache && cache_s, "smh_kv_fork: null pointer");
    long v1 = row_bytes / 16, v2 = row_scales * 2 / 16;
    hipLaunchKernelGGL(kv_fork_kernel, dim3((unsigned)((v1 + 255) / 256), forks), dim3(256), 0, (hipStream_t)stream,
                       (u32x4 *)cache, v1, origin, curr);
    hipLaunchKernelGGL(kv_fork_kernel, dim3((unsigned)((v2 + 255) / 256), forks), dim3(256), 0, (hipStream_t)stream,
                       (u32x4 *)cache_s, v2, origin, curr);
    return launch_status();
}
