// Consumers of the Q4_0 matmul's K-slice slabs.
//
// The matmul kernels leave `ksplit` slabs partial[s][m][n] (fp32);
// every kernel here first forms acc = sum_s partial[s][m][n] in fp32 (slice order, so the result does not depend on scheduling), rounds
// it ONCE to fp16 - the value the reference's matmul_q40 returns - and then applies the operator
// that follows the linear in the model:
//   partial_reduce_kernel      c = fp16(acc) (+ fp16 residual add)
//   partial_rmsnorm_kernel     h = h_in + fp16(acc);  xn = RMSNorm(h) * weight
//   partial_silu_mul_kernel    out = fp16(silu(fp16(acc_gate))) * fp16(acc_up)
//   partial_rope_append_kernel q,k,v = fp16(acc); RoPE(q,k); Q4_0 append of k,v to the suffix cache
// so a decode layer is 4 weight-streaming launches plus these small ones, and no kernel ever waits
// for another workgroup.
#include "q40_matmul.hpp"
#include "rope_kv.hpp"
#include "slab_sum.hpp"

namespace smh {

// ---- plain reduce (+ residual) ------------------------------------------------------------------
__global__ __launch_bounds__(256) void partial_reduce_kernel(const void *__restrict__ partial, int ksplit, int M, int n_total,
                                                             int col0, int N, half_t *__restrict__ c, long ldc, int epilogue,
                                                             const half_t *__restrict__ resid, long ldr) {
    const long i = ((long)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= (long)M * N) return;
    const int m = (int)(i / N), n = (int)(i % N);          // N % 4 == 0: the 4 columns share a row
    const f4 acc = slab_sum4(partial, (long)m * n_total + col0 + n, (long)M * n_total, ksplit);
    h4 out;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        half_t v = (half_t)acc[j];
        if (epilogue == SMH_EPI_RESIDUAL) v = (half_t)((float)resid[(long)m * ldr + n + j] + (float)v);
        out[j] = v;
    }
    *reinterpret_cast<h4 *>(c + (long)m * ldc + n) = out;
}

// ---- residual add + RMSNorm ---------------------------------------------------------------------
// one workgroup of 1024 threads per row; h_out = h_in + fp16(acc) (fp16 add), xn = fp16(fp16(h*r)*w)
__global__ __launch_bounds__(1024) void partial_rmsnorm_kernel(const void *__restrict__ partial, int ksplit, int M, int N,
                                                               const half_t *__restrict__ h_in, const half_t *__restrict__ wt,
                                                               float eps, half_t *__restrict__ h_out, half_t *__restrict__ xn_out) {
    __shared__ float s_part[16];
    const int m = blockIdx.x;
    const long slab = (long)M * N;
    float ss = 0.f;
    // each thread owns columns 4t, 4t+1, 4t+2, 4t+3 (+ 4096 per pass); values kept for the second pass
    constexpr int MAXPASS = 4;      // N <= 16384
    h4 hv[MAXPASS], wv[MAXPASS];
    // the norm weights are not needed before the second pass: fetched now, they arrive with the slabs
#pragma unroll
    for (int ps = 0; ps < MAXPASS; ++ps) {
        const int n = (ps * 1024 + threadIdx.x) * 4;
        if (n < N) wv[ps] = *reinterpret_cast<const h4 *>(wt + n);
    }
#pragma unroll
    for (int ps = 0; ps < MAXPASS; ++ps) {
        const int n = (ps * 1024 + threadIdx.x) * 4;
        if (n < N) {
            h4 v;
            if (partial != nullptr) {
                const f4 acc = slab_sum4(partial, (long)m * N + n, slab, ksplit);
#pragma unroll
                for (int j = 0; j < 4; ++j) v[j] = (half_t)acc[j];
                if (h_in != nullptr) {
                    const h4 r = *reinterpret_cast<const h4 *>(h_in + (long)m * N + n);
#pragma unroll
                    for (int j = 0; j < 4; ++j) v[j] = (half_t)((float)r[j] + (float)v[j]);
                }
            } else {
                v = *reinterpret_cast<const h4 *>(h_in + (long)m * N + n);
            }
            hv[ps] = v;
            if (h_out != nullptr) *reinterpret_cast<h4 *>(h_out + (long)m * N + n) = v;
#pragma unroll
            for (int j = 0; j < 4; ++j) ss = sumsq_add(ss, (float)v[j]);
        }
    }
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = ss;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < 16; ++w) total += s_part[w];
    const float r = rms_factor(total, N, eps);
#pragma unroll
    for (int ps = 0; ps < MAXPASS; ++ps) {
        const int n = (ps * 1024 + threadIdx.x) * 4;
        if (n < N) {
            const h4 w = wv[ps];
            h4 o;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                half_t nv = scale_to_half(hv[ps][j], r);
                o[j] = nv * w[j];
            }
            *reinterpret_cast<h4 *>(xn_out + (long)m * N + n) = o;
        }
    }
}

// ---- residual add + sums of squares (the first half of partial_rmsnorm_kernel, spread over 16 workgroups a row) ----
// grid (16, M), one wave each: wave w of a row is wave w of partial_rmsnorm_kernel's workgroup (same columns per
// thread, same order of additions), so sums[m][0..15] added in index order give that kernel's sum of squares bit
// for bit.  The consumer (the matmul that follows, q40_gemv_kernel LAYOUT 3) normalises its own K-slice.
__global__ __launch_bounds__(64) void partial_residual_sumsq_kernel(const void *__restrict__ partial, int ksplit, int M, int N,
                                                                    const half_t *__restrict__ h_in, half_t *__restrict__ h_out,
                                                                    float *__restrict__ sums) {
    const int m = blockIdx.y;
    const int vt = blockIdx.x * 64 + threadIdx.x;      // thread index inside partial_rmsnorm_kernel's workgroup
    const long slab = (long)M * N;
    constexpr int MAXPASS = 4;      // N <= 16384
    f4 acc[MAXPASS];
    h4 res[MAXPASS];
#pragma unroll
    for (int ps = 0; ps < MAXPASS; ++ps) {
        const int n = (ps * 1024 + vt) * 4;
        if (n < N) {
            acc[ps] = slab_sum4(partial, (long)m * N + n, slab, ksplit);
            if (h_in != nullptr) res[ps] = *reinterpret_cast<const h4 *>(h_in + (long)m * N + n);
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int ps = 0; ps < MAXPASS; ++ps) {
        const int n = (ps * 1024 + vt) * 4;
        if (n < N) {
            h4 v;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                v[j] = (half_t)acc[ps][j];
                if (h_in != nullptr) v[j] = (half_t)((float)res[ps][j] + (float)v[j]);
            }
            *reinterpret_cast<h4 *>(h_out + (long)m * N + n) = v;
#pragma unroll
            for (int j = 0; j < 4; ++j) ss = sumsq_add(ss, (float)v[j]);
        }
    }
    ss = wave_sum(ss);
    if (threadIdx.x == 0) sums[(long)m * SMH_NORM_SUMS + blockIdx.x] = ss;
}

// ---- SwiGLU gate ------------------------------------------------------------------------------------
// slabs hold [gate | up] (2 * n_half columns)
__global__ __launch_bounds__(256) void partial_silu_mul_kernel(const void *__restrict__ partial, int ksplit, int M, int n_half,
                                                               half_t *__restrict__ out) {
    // grid (quads of a row, rows): no division to find the row (a 64-bit one costs more than the rest of the arithmetic)
    const int m = blockIdx.y, n = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (n >= n_half) return;
    const long slab = (long)M * 2 * n_half;
    const f4 ga = slab_sum4(partial, (long)m * 2 * n_half + n, slab, ksplit);
    const f4 ua = slab_sum4(partial, (long)m * 2 * n_half + n_half + n, slab, ksplit);
    h4 o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float gf = (float)(half_t)ga[j];
        const half_t sl = (half_t)(gf / (1.0f + expf(-gf)));
        o[j] = sl * (half_t)ua[j];
    }
    *reinterpret_cast<h4 *>(out + (long)m * n_half + n) = o;
}

// one wave per (branch, head); heads 0..H-1 queries, H..H+Hkv-1 keys, H+Hkv.. values.
// slab columns: [q (H*128) | k (Hkv*128) | v (Hkv*128)]
__global__ __launch_bounds__(256) void partial_rope_append_kernel(const void *__restrict__ partial, int ksplit, int B, int H, int Hkv,
                                                                  half_t *__restrict__ q, half_t *__restrict__ k, half_t *__restrict__ v,
                                                                  const half_t *__restrict__ cos_tab, const half_t *__restrict__ sin_tab,
                                                                  const int32_t *__restrict__ pos_dev,
                                                                  uint8_t *__restrict__ cache_k, half_t *__restrict__ cache_ks,
                                                                  uint8_t *__restrict__ cache_v, half_t *__restrict__ cache_vs,
                                                                  int Smax, const int32_t *__restrict__ t_dev) {
    __shared__ float s_row[4][128];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    // grid (groups of four heads, branches)
    const int heads = H + 2 * Hkv;
    const int hh = blockIdx.x * 4 + wave;
    const bool live = hh < heads;
    const int b = blockIdx.y;
    const int h = live ? hh : 0;
    const int n_total = heads * 128;
    // the slabs are read two adjacent columns per lane; the rotation pairs column i with i + 64, so the sums
    // change lanes through LDS
    // the position and the rotation factors travel while the slabs are read
    const int t = (t_dev != nullptr) ? *t_dev : -1;
    const int pos = *pos_dev;
    const half_t cos_l = cos_tab[(long)pos * 64 + lane], sin_l = sin_tab[(long)pos * 64 + lane];
    if (live) {
        const f2 sum = slab_sum2(partial, (long)b * n_total + (long)h * 128 + 2 * lane, (long)B * n_total, ksplit);
        *reinterpret_cast<f2 *>(&s_row[wave][2 * lane]) = sum;
    }
    __syncthreads();
    if (!live) return;
    half_t x1 = (half_t)s_row[wave][lane];
    half_t x2 = (half_t)s_row[wave][lane + 64];
    if (h >= H + Hkv) {                                      // value head: store, append
        const int hk = h - H - Hkv;
        half_t *pv = v + ((long)b * Hkv + hk) * 128;
        pv[lane] = x1;
        pv[lane + 64] = x2;
        if (cache_v != nullptr && t >= 0 && t < Smax) {
            const long row = ((long)b * Smax + t) * Hkv + hk;
            kv_store_row2(x1, x2, cache_v + row * 64, cache_vs + row * 2, lane);
        }
        return;
    }
    rope_pair2(x1, x2, cos_l, sin_l);
    if (h < H) {
        half_t *pq = q + ((long)b * H + h) * 128;
        pq[lane] = x1;
        pq[lane + 64] = x2;
        return;
    }
    const int hk = h - H;
    half_t *pk = k + ((long)b * Hkv + hk) * 128;
    pk[lane] = x1;
    pk[lane + 64] = x2;
    if (cache_k != nullptr && t >= 0 && t < Smax) {
        const long row = ((long)b * Smax + t) * Hkv + hk;
        kv_store_row2(x1, x2, cache_k + row * 64, cache_ks + row * 2, lane);
    }
}

}  // namespace smh

using namespace smh;

// ---- host side: plan, produce, consume ----------------------------------------------------------------
static int fill_params(MatmulParams &p, const void *a, int M, int K, long lda, int nseg, const void *const *w,
                       const void *const *s, const int *n, const char *who, bool tiled = false) {
    SMH_REQUIRE(M >= 0, "%s: M=%d", who, M);
    SMH_REQUIRE(K > 0 && K % 8 == 0, "%s: K=%d must be a positive multiple of 8", who, K);
    SMH_REQUIRE(nseg >= 1 && nseg <= SMH_MAX_SEGMENTS && n != nullptr, "%s: nseg=%d outside [1,%d]", who, nseg, SMH_MAX_SEGMENTS);
    SMH_REQUIRE(lda >= K && lda % 8 == 0, "%s: lda=%ld must be >= K and a multiple of 8 (128-bit loads)", who, lda);
    p = MatmulParams{};
    p.a = (const half_t *)a;
    p.M = M; p.K = K; p.lda = lda; p.nseg = nseg;
    for (int i = 0; i < nseg; ++i) {
        SMH_REQUIRE(n[i] > 0 && n[i] % 128 == 0, "%s: N=%d must be a positive multiple of 128", who, n[i]);
        p.seg[i].w = w ? (const uint8_t *)w[i] : nullptr;
        p.seg[i].s = s ? (const half_t *)s[i] : nullptr;
        p.seg[i].N = n[i];
    }
    p.tiled = tiled ? 1 : 0;                   // (the plan above 16 rows depends on the layout)
    if (M <= SMH_GEMV_MAX_M) gemv_fill_plan(p); else gemm_fill_plan(p);
    return 0;
}

extern "C" int smh_q40_matmul_plan(int M, int K, int nseg, const int *n) {
    MatmulParams p;
    if (M <= 0) return 1;
    int st = fill_params(p, nullptr, M, K, (K + 7) / 8 * 8, nseg, nullptr, nullptr, n, "smh_q40_matmul_plan");
    return st < 0 ? st : p.ksplit;
}

extern "C" int smh_q40_swiglu_fits(int M, int K, int n_half) { return smh::gemm_swiglu_fits(M, K, n_half, true) ? 1 : 0; }

extern "C" int smh_q40_matmul_tiled_swiglu(const void *a, int M, int K, long lda, const void *tiled_gate, const void *tiled_up, int n_half,
                                           void *out, long ldo, smh_stream_t stream) {
    const char *who = "smh_q40_matmul_tiled_swiglu";
    SMH_REQUIRE(gemm_swiglu_fits(M, K, n_half, false),
                "%s: M=%d (17 .. 128) K=%d (a multiple of 64) n_half=%d (a multiple of 128, at most 16384)", who, M, K, n_half);
    SMH_REQUIRE(a && tiled_gate && tiled_up && out, "%s: null pointer", who);
    SMH_REQUIRE(lda >= K && lda % 8 == 0 && ldo >= n_half && ldo % 2 == 0, "%s: lda=%ld (>= K, a multiple of 8) ldo=%ld (>= n_half, even)", who, lda, ldo);
    SMH_REQUIRE(((uintptr_t)a & 15) == 0 && ((uintptr_t)out & 3) == 0 && ((uintptr_t)tiled_gate & 127) == 0 && ((uintptr_t)tiled_up & 127) == 0,
                "%s: misaligned pointer", who);
    MatmulParams p = MatmulParams{};
    p.a = (const half_t *)a; p.M = M; p.K = K; p.lda = lda; p.nseg = 2;
    p.seg[0].w = (const uint8_t *)tiled_gate; p.seg[0].N = n_half;
    p.seg[1].w = (const uint8_t *)tiled_up; p.seg[1].N = n_half;
    p.c = (half_t *)out; p.ldc = ldo; p.tiled = 1;
    return gemm_swiglu_launch(p, (hipStream_t)stream);
}

extern "C" int smh_q40_matmul_plan_tiled(int M, int K, int nseg, const int *n) {
    MatmulParams p;
    if (M <= 0) return 1;
    int st = fill_params(p, nullptr, M, K, (K + 7) / 8 * 8, nseg, nullptr, nullptr, n, "smh_q40_matmul_plan_tiled", true);
    return st < 0 ? st : p.ksplit;
}

extern "C" size_t smh_q40_matmul_workspace_bytes(int max_m, int max_n) {
    // K is split only while (column units x row blocks) <= 512, so the slabs never exceed
    // 512 tiles of 128 x 256 floats for the GEMM, or SMH_MAX_KSPLIT x 16 x N floats for the GEMV
    size_t n = (size_t)(max_n < 128 ? 128 : max_n);
    size_t m = (size_t)(max_m < 1 ? 1 : (max_m > SMH_GEMV_MAX_M ? SMH_GEMV_MAX_M : max_m));
    size_t floats = n * m * SMH_MAX_KSPLIT;
    if (max_m > SMH_GEMV_MAX_M && floats < (size_t)512 * 128 * 256) floats = (size_t)512 * 128 * 256;
    return floats * sizeof(float) + 256;
}

extern "C" int smh_q40_matmul_partial(const void *a, int M, int K, long lda, int nseg, const void *const *w,
                                      const void *const *s, const int *n, void *partial, size_t partial_bytes,
                                      smh_stream_t stream) {
    MatmulParams p;
    int st = fill_params(p, a, M, K, lda, nseg, w, s, n, "smh_q40_matmul_partial");
    if (st) return st;
    if (M == 0) return 0;
    SMH_REQUIRE(a && w && s && partial, "smh_q40_matmul_partial: null pointer");
    for (int i = 0; i < nseg; ++i) SMH_REQUIRE(w[i] && s[i], "smh_q40_matmul_partial: null weight %d", i);
    size_t need = (size_t)p.ksplit * M * p.n_total * sizeof(float);
    SMH_REQUIRE(partial_bytes >= need, "smh_q40_matmul_partial: partial buffer %zu < %zu bytes", partial_bytes, need);
    p.partial = (float *)partial;
    p.direct = 0;
    return M <= SMH_GEMV_MAX_M ? gemv_launch(p, (hipStream_t)stream) : gemm_launch(p, (hipStream_t)stream);
}

extern "C" int smh_q40_matmul_partial_tiled(const void *a, int M, int K, long lda, int nseg, const void *const *tiled,
                                            const int *n, void *partial, size_t partial_bytes, smh_stream_t stream) {
    MatmulParams p;
    int st = fill_params(p, a, M, K, lda, nseg, tiled, nullptr, n, "smh_q40_matmul_partial_tiled", true);
    if (st) return st;
    if (M == 0) return 0;
    SMH_REQUIRE(a && tiled && partial, "smh_q40_matmul_partial_tiled: null pointer");
    for (int i = 0; i < nseg; ++i)
        SMH_REQUIRE(tiled[i] && ((uintptr_t)tiled[i] & 127) == 0, "smh_q40_matmul_partial_tiled: weight %d is null or not 128-byte aligned", i);
    size_t need = (size_t)p.ksplit * M * p.n_total * sizeof(float);
    SMH_REQUIRE(partial_bytes >= need, "smh_q40_matmul_partial_tiled: partial buffer %zu < %zu bytes", partial_bytes, need);
    p.partial = (float *)partial;
    p.direct = 0;
    p.tiled = 1;
    return M <= SMH_GEMV_MAX_M ? gemv_launch(p, (hipStream_t)stream) : gemm_launch(p, (hipStream_t)stream);
}

extern "C" int smh_q40_matmul_partial_tiled_silu(const void *gate_up_partial, int gate_up_ksplit, int M, int K, int nseg,
                                                 const void *const *tiled, const int *n, void *partial, size_t partial_bytes,
                                                 smh_stream_t stream) {
    MatmulParams p;
    int st = fill_params(p, nullptr, M, K, (K + 7) / 8 * 8, nseg, tiled, nullptr, n, "smh_q40_matmul_partial_tiled_silu", true);
    if (st) return st;
    if (M == 0) return 0;
    SMH_REQUIRE(M <= SMH_SILU_IN_MAX_M, "smh_q40_matmul_partial_tiled_silu: M=%d (at most %d rows; use smh_partial_silu_mul above)", M, SMH_SILU_IN_MAX_M);
    SMH_REQUIRE(K % 32 == 0, "smh_q40_matmul_partial_tiled_silu: K=%d must be a multiple of 32", K);
    SMH_REQUIRE(gate_up_partial && tiled && partial, "smh_q40_matmul_partial_tiled_silu: null pointer");
    SMH_REQUIRE(gate_up_ksplit >= 1 && gate_up_ksplit <= SMH_MAX_KSPLIT, "smh_q40_matmul_partial_tiled_silu: ksplit=%d", gate_up_ksplit);
    for (int i = 0; i < nseg; ++i)
        SMH_REQUIRE(tiled[i] && ((uintptr_t)tiled[i] & 127) == 0, "smh_q40_matmul_partial_tiled_silu: weight %d is null or not 128-byte aligned", i);
    size_t need = (size_t)p.ksplit * M * p.n_total * sizeof(float);
    SMH_REQUIRE(partial_bytes >= need, "smh_q40_matmul_partial_tiled_silu: partial buffer %zu < %zu bytes", partial_bytes, need);
    SMH_REQUIRE(partial != gate_up_partial, "smh_q40_matmul_partial_tiled_silu: the product cannot overwrite the slabs it is made from");
    p.partial = (float *)partial;
    p.direct = 0;
    p.tiled = 1;
    p.gu_partial = (const float *)gate_up_partial;
    p.gu_ksplit = gate_up_ksplit;
    return gemv_launch(p, (hipStream_t)stream);
}

extern "C" int smh_q40_norm_in_fits(int M, int K, int nseg, const int *n) {
    MatmulParams p;
    if (M <= 0 || M > SMH_GEMV_MAX_M || K % 32 != 0) return 0;
    int st = fill_params(p, nullptr, M, K, (K + 7) / 8 * 8, nseg, nullptr, nullptr, n, "smh_q40_norm_in_fits", true);
    return st < 0 ? st : (gemv_norm_in_fits(p) ? 1 : 0);
}

extern "C" int smh_q40_matmul_partial_tiled_norm(const void *h, long ldh, const void *sums, const void *norm_weight, float eps,
                                                 int M, int K, int nseg, const void *const *tiled, const int *n,
                                                 void *partial, size_t partial_bytes, smh_stream_t stream) {
    const char *who = "smh_q40_matmul_partial_tiled_norm";
    MatmulParams p;
    int st = fill_params(p, h, M, K, ldh, nseg, tiled, nullptr, n, who, true);
    if (st) return st;
    if (M == 0) return 0;
    SMH_REQUIRE(M <= SMH_GEMV_MAX_M, "%s: M=%d (at most %d rows; use smh_partial_rmsnorm above)", who, M, SMH_GEMV_MAX_M);
    SMH_REQUIRE(K % 32 == 0 && ldh % 8 == 0, "%s: K=%d must be a multiple of 32, ldh=%ld of 8", who, K, ldh);
    SMH_REQUIRE(h && sums && norm_weight && tiled && partial, "%s: null pointer", who);
    SMH_REQUIRE(((uintptr_t)h & 15) == 0 && ((uintptr_t)norm_weight & 15) == 0 && ((uintptr_t)sums & 15) == 0, "%s: h, norm_weight and sums must be 16-byte aligned", who);
    for (int i = 0; i < nseg; ++i)
        SMH_REQUIRE(tiled[i] && ((uintptr_t)tiled[i] & 127) == 0, "%s: weight %d is null or not 128-byte aligned", who, i);
    SMH_REQUIRE(gemv_norm_in_fits(p), "%s: %d rows x K-slices of %d rows exceed %d bytes (ask smh_q40_norm_in_fits first)", who, M,
                p.steps_per_slice * 32, SMH_NORM_IN_MAX_XS_BYTES);
    size_t need = (size_t)p.ksplit * M * p.n_total * sizeof(float);
    SMH_REQUIRE(partial_bytes >= need, "%s: partial buffer %zu < %zu bytes", who, partial_bytes, need);
    p.partial = (float *)partial;
    p.direct = 0;
    p.tiled = 1;
    p.norm_w = (const half_t *)norm_weight;
    p.norm_ss = (const float *)sums;
    p.norm_eps = eps;
    return gemv_launch(p, (hipStream_t)stream);
}

static int reduce_launch(const void *partial, int ksplit, int M, int n_total, int col0, int N, void *c, long ldc,
                         int epilogue, const void *residual, long ldr, hipStream_t stream) {
    long quads = ((long)M * N + 3) / 4;
    hipLaunchKernelGGL(partial_reduce_kernel, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, stream,
                       partial, ksplit, M, n_total, col0, N, (half_t *)c, ldc, epilogue, (const half_t *)residual, ldr);
    return launch_status();
}

extern "C" int smh_partial_reduce(const void *partial, int ksplit, int M, int n_total, int col0, int N, void *c, long ldc,
                                  int epilogue, const void *residual, long ldr, smh_stream_t stream) {
    SMH_REQUIRE(ksplit >= 1 && ksplit <= SMH_MAX_KSPLIT, "smh_partial_reduce: ksplit=%d outside [1,%d]", ksplit, SMH_MAX_KSPLIT);
    SMH_REQUIRE(M >= 0 && N > 0 && N % 4 == 0 && col0 >= 0 && col0 % 4 == 0 && col0 + N <= n_total && n_total % 4 == 0,
                "smh_partial_reduce: M=%d N=%d col0=%d n_total=%d", M, N, col0, n_total);
    SMH_REQUIRE(epilogue == SMH_EPI_NONE || epilogue == SMH_EPI_RESIDUAL, "smh_partial_reduce: epilogue=%d", epilogue);
    if (M == 0) return 0;
    SMH_REQUIRE(partial && c && ldc >= N && ldc % 4 == 0, "smh_partial_reduce: bad output");
    SMH_REQUIRE(epilogue != SMH_EPI_RESIDUAL || (residual && ldr >= N), "smh_partial_reduce: residual missing");
    return reduce_launch(partial, ksplit, M, n_total, col0, N, c, ldc, epilogue, residual, ldr, (hipStream_t)stream);
}

static int matmul_fp16(const void *a, int M, int K, long lda, const void *b_w, const void *b_s, int N, void *c, long ldc,
                       int epilogue, const void *residual, long ldr, void *workspace, size_t workspace_bytes,
                       smh_stream_t stream, const char *who, int force) {
    SMH_REQUIRE(force != 1 || M <= SMH_GEMV_MAX_M, "%s: M=%d outside [0,%d]", who, M, SMH_GEMV_MAX_M);
    SMH_REQUIRE(epilogue == SMH_EPI_NONE || epilogue == SMH_EPI_RESIDUAL, "%s: epilogue=%d", who, epilogue);
    SMH_REQUIRE(ldc >= N, "%s: ldc=%ld too small", who, ldc);
    MatmulParams p;
    const void *ws[1] = {b_w};
    const void *ss[1] = {b_s};
    int st = fill_params(p, a, M, K, lda, 1, ws, ss, &N, who);
    if (st) return st;
    if (M == 0) return 0;
    SMH_REQUIRE(a && b_w && b_s && c, "%s: null pointer", who);
    SMH_REQUIRE(epilogue != SMH_EPI_RESIDUAL || (residual && ldr >= N), "%s: residual missing", who);
    if (force == 2 && M <= SMH_GEMV_MAX_M) gemm_fill_plan(p);        // smh_q40_gemm on a small batch
    const bool gemm = (force == 2) || M > SMH_GEMV_MAX_M;
    p.c = (half_t *)c; p.ldc = ldc; p.resid = (const half_t *)residual; p.ldr = ldr; p.epilogue = epilogue;
    if (p.ksplit == 1) {
        p.direct = 1;
        SMH_REQUIRE(!gemm || ldc % 8 == 0, "%s: ldc=%ld must be a multiple of 8 for M > 16", who, ldc);
        return gemm ? gemm_launch(p, (hipStream_t)stream) : gemv_launch(p, (hipStream_t)stream);
    }
    size_t need = (size_t)p.ksplit * M * N * sizeof(float);
    SMH_REQUIRE(workspace && workspace_bytes >= need, "%s: workspace %zu < %zu bytes", who, workspace_bytes, need);
    p.partial = (float *)workspace;
    p.direct = 0;
    st = gemm ? gemm_launch(p, (hipStream_t)stream) : gemv_launch(p, (hipStream_t)stream);
    if (st) return st;
    SMH_REQUIRE(ldc % 4 == 0, "%s: ldc=%ld must be a multiple of 4", who, ldc);
    return reduce_launch(p.partial, p.ksplit, M, N, 0, N, c, ldc, epilogue, residual, ldr, (hipStream_t)stream);
}

extern "C" int smh_q40_gemv(const void *a, int M, int K, long lda, const void *b_w, const void *b_s, int N, void *c, long ldc,
                            int epilogue, const void *residual, long ldr, void *workspace, size_t workspace_bytes, smh_stream_t stream) {
    return matmul_fp16(a, M, K, lda, b_w, b_s, N, c, ldc, epilogue, residual, ldr, workspace, workspace_bytes, stream, "smh_q40_gemv", 1);
}
extern "C" int smh_q40_gemm(const void *a, int M, int K, long lda, const void *b_w, const void *b_s, int N, void *c, long ldc,
                            int epilogue, const void *residual, long ldr, void *workspace, size_t workspace_bytes, smh_stream_t stream) {
    return matmul_fp16(a, M, K, lda, b_w, b_s, N, c, ldc, epilogue, residual, ldr, workspace, workspace_bytes, stream, "smh_q40_gemm", 2);
}
extern "C" int smh_q40_matmul(const void *a, int M, int K, long lda, const void *b_w, const void *b_s, int N, void *c, long ldc,
                              int epilogue, const void *residual, long ldr, void *workspace, size_t workspace_bytes, smh_stream_t stream) {
    return matmul_fp16(a, M, K, lda, b_w, b_s, N, c, ldc, epilogue, residual, ldr, workspace, workspace_bytes, stream, "smh_q40_matmul", 0);
}

extern "C" int smh_partial_rmsnorm(const void *partial, int ksplit, int M, int N, const void *h_in, const void *weight, float eps,
                                   void *h_out, void *xn_out, smh_stream_t stream) {
    SMH_REQUIRE(partial == nullptr || (ksplit >= 1 && ksplit <= SMH_MAX_KSPLIT), "smh_partial_rmsnorm: ksplit=%d", ksplit);
    SMH_REQUIRE(M >= 0 && N > 0 && N % 4 == 0 && N <= 16384, "smh_partial_rmsnorm: M=%d N=%d (N must be a multiple of 4, <= 16384)", M, N);
    SMH_REQUIRE(partial != nullptr || h_in != nullptr, "smh_partial_rmsnorm: no input");
    if (M == 0) return 0;
    SMH_REQUIRE(weight && xn_out, "smh_partial_rmsnorm: null pointer");
    hipLaunchKernelGGL(partial_rmsnorm_kernel, dim3(M), dim3(1024), 0, (hipStream_t)stream, partial, ksplit, M, N,
                       (const half_t *)h_in, (const half_t *)weight, eps, (half_t *)h_out, (half_t *)xn_out);
    return launch_status();
}

extern "C" int smh_partial_residual_sumsq(const void *partial, int ksplit, int M, int N, const void *h_in, void *h_out, void *sums,
                                          smh_stream_t stream) {
    SMH_REQUIRE(partial != nullptr && ksplit >= 1 && ksplit <= SMH_MAX_KSPLIT, "smh_partial_residual_sumsq: partial=%p ksplit=%d", partial, ksplit);
    SMH_REQUIRE(M >= 0 && N > 0 && N % 4 == 0 && N <= 16384, "smh_partial_residual_sumsq: M=%d N=%d (N must be a multiple of 4, <= 16384)", M, N);
    if (M == 0) return 0;
    SMH_REQUIRE(h_out && sums, "smh_partial_residual_sumsq: null pointer");
    hipLaunchKernelGGL(partial_residual_sumsq_kernel, dim3(SMH_NORM_SUMS, M), dim3(64), 0, (hipStream_t)stream, partial, ksplit, M, N,
                       (const half_t *)h_in, (half_t *)h_out, (float *)sums);
    return launch_status();
}

extern "C" int smh_partial_silu_mul(const void *partial, int ksplit, int M, int n_half, void *out, smh_stream_t stream) {
    SMH_REQUIRE(ksplit >= 1 && ksplit <= SMH_MAX_KSPLIT, "smh_partial_silu_mul: ksplit=%d", ksplit);
    SMH_REQUIRE(M >= 0 && n_half > 0 && n_half % 4 == 0, "smh_partial_silu_mul: M=%d n_half=%d", M, n_half);
    if (M == 0) return 0;
    SMH_REQUIRE(partial && out, "smh_partial_silu_mul: null pointer");
    SMH_REQUIRE(M <= 65535, "smh_partial_silu_mul: M=%d (at most 65535 rows per launch)", M);
    hipLaunchKernelGGL(partial_silu_mul_kernel, dim3((unsigned)((n_half / 4 + 255) / 256), (unsigned)M), dim3(256), 0, (hipStream_t)stream,
                       partial, ksplit, M, n_half, (half_t *)out);
    return launch_status();
}

extern "C" int smh_partial_rope_append_kv(const void *partial, int ksplit, int B, int H, int Hkv, int D, void *q, void *k, void *v,
                                          const void *cos_tab, const void *sin_tab, const int32_t *pos_dev,
                                          void *cache_k, void *cache_ks, void *cache_v, void *cache_vs, int Smax,
                                          const int32_t *t_dev, smh_stream_t stream) {
    SMH_REQUIRE(D == 128, "smh_partial_rope_append_kv: head dim %d (only 128)", D);
    SMH_REQUIRE(ksplit >= 1 && ksplit <= SMH_MAX_KSPLIT, "smh_partial_rope_append_kv: ksplit=%d", ksplit);
    SMH_REQUIRE(B >= 0 && H > 0 && Hkv > 0, "smh_partial_rope_append_kv: B=%d H=%d Hkv=%d", B, H, Hkv);
    if (B == 0) return 0;
    SMH_REQUIRE(partial && q && k && v && cos_tab && sin_tab && pos_dev, "smh_partial_rope_append_kv: null pointer");
    SMH_REQUIRE(!cache_k || (cache_ks && cache_v && cache_vs && t_dev && Smax > 0), "smh_partial_rope_append_kv: cache arguments incomplete");
    SMH_REQUIRE(B <= 65535, "smh_partial_rope_append_kv: B=%d (at most 65535 branches per launch)", B);
    hipLaunchKernelGGL(partial_rope_append_kernel, dim3((unsigned)((H + 2 * Hkv + 3) / 4), (unsigned)B), dim3(256), 0, (hipStream_t)stream,
                       partial, ksplit, B, H, Hkv, (half_t *)q, (half_t *)k, (half_t *)v,
                       (const half_t *)cos_tab, (const half_t *)sin_tab, pos_dev, (uint8_t *)cache_k, (half_t *)cache_ks,
                       (uint8_t *)cache_v, (half_t *)cache_vs, Smax, t_dev);
    return launch_status();
}
