// Finishing a Q4_0 matmul inside the matmul kernel itself.
//
// The matmul kernels cut K into slices; each (column unit, slice) workgroup leaves an fp32 partial
// [M, 256].  With a finisher the workgroup then counts its arrival on the unit's counter, and the arrival
// that completes the unit adds the partials in slice order (the result does not depend on timing), rounds
// once to fp16 - the value the reference's matmul_q40 returns - and applies the operator that follows the
// linear in the model, instead of leaving that to another launch:
//   STORE            c = fp16(sum) (+ fp16 residual add)
//   RESIDUAL_RMSNORM h = h_in + fp16(sum); when the last UNIT of the matrix is done, that workgroup also
//                    forms xn = RMSNorm(h) * weight for all rows (second-level counter)
//   SILU_MUL         act = fp16(silu(fp16(sum_gate))) * fp16(sum_up); gate unit j and up unit j share a counter
//   ROPE_APPEND      q,k,v = fp16(sum); RoPE(q,k); Q4_0 append of k,v to the branch's suffix cache
// Nothing waits: a workgroup that is not last simply ends.  Partials and everything a later finisher
// of the same launch reads are written with coherent stores.
#pragma once

#include "rope_kv.hpp"
#include "smh_common.hpp"

namespace smh {

struct MatmulFinish {
    int mode;                       // SMH_FIN_*
    uint32_t *unit_cnt;             // [units] (pairs for SILU_MUL), zero between launches
    uint32_t *row_cnt;              // RESIDUAL_RMSNORM: one counter over the units
    half_t *out;                    // STORE: c [M, ldo]; SILU_MUL: act [M, ldo]
    long ldo;
    const half_t *resid;            // STORE (optional), RESIDUAL_RMSNORM: h_in [M, ldr]
    long ldr;
    half_t *h_out;                  // RESIDUAL_RMSNORM: h [M, N]
    float *ssq;                     // RESIDUAL_RMSNORM: [units][M] sums of squares
    const half_t *norm_w;
    half_t *xn_out;                 // [M, N]
    float eps;
    // ROPE_APPEND (columns: q heads | k heads | v heads, 128 wide)
    int H, Hkv, Smax;
    half_t *q, *k, *v;
    const half_t *cos_tab, *sin_tab;
    const int32_t *pos_dev, *t_dev;
    uint8_t *cache_k, *cache_v;
    half_t *cache_ks, *cache_vs;
};

// sum over the K-slices of 4 / 1 consecutive columns of row m (loads issued together)
__device__ __forceinline__ f4 slices_sum4(const float *p, long slab_stride, int ksplit) {
    f4 v[SMH_MAX_KSPLIT];
#pragma unroll
    for (int s = 0; s < SMH_MAX_KSPLIT; ++s) v[s] = (s < ksplit) ? ld_f4(p + s * slab_stride) : f4{0.f, 0.f, 0.f, 0.f};
    f4 tot = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < SMH_MAX_KSPLIT; ++s) tot += v[s];
    return tot;
}
__device__ __forceinline__ float slices_sum1(const float *p, long slab_stride, int ksplit) {
    float v[SMH_MAX_KSPLIT];
#pragma unroll
    for (int s = 0; s < SMH_MAX_KSPLIT; ++s) v[s] = (s < ksplit) ? ld_f32(p + s * slab_stride) : 0.f;
    float tot = 0.f;
#pragma unroll
    for (int s = 0; s < SMH_MAX_KSPLIT; ++s) tot += v[s];
    return tot;
}

// Called by all threads of the workgroup after its partial has been written (coherent stores).
// `n0`: first column of the unit in the concatenated output, `width` <= 256 valid columns,
// `unit`: index over all segments, `units`: their number, `seg`/`n_seg0`: segment and column inside it.
// Returns after the finisher work, if any, is complete.
template <int THREADS>
__device__ __forceinline__ void matmul_finish(const MatmulFinish &f, const float *partial, int ksplit, int M, int n_total,
                                              int unit, int units, int n0, int width, int seg, int n_seg0, uint32_t *s_flag) {
    constexpr int WAVES = THREADS / 64;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const long slab = (long)M * n_total;
    int cu = unit;
    uint32_t expected = (uint32_t)ksplit;
    if (f.mode == SMH_FIN_SILU_MUL) {
        const int half = units / 2;
        cu = unit >= half ? unit - half : unit;
        expected *= 2u;
    }
    wait_vmem();
    __syncthreads();
    if (tid == 0) {
        const uint32_t prev = __hip_atomic_fetch_add(f.unit_cnt + cu, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const bool last = prev == expected - 1u;
        if (last) st_u32(f.unit_cnt + cu, 0u);
        *s_flag = last ? 1u : 0u;
    }
    __syncthreads();
    if (*s_flag == 0u) return;

    if (f.mode == SMH_FIN_STORE) {
        for (int i = tid; i < M * 64; i += THREADS) {
            const int m = i >> 6, c4 = 4 * (i & 63);
            if (c4 >= width) continue;
            const f4 acc = slices_sum4(partial + (long)m * n_total + n0 + c4, slab, ksplit);
            h4 o;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                half_t v = (half_t)acc[j];
                if (f.resid != nullptr) v = (half_t)((float)f.resid[(long)m * f.ldr + n0 + c4 + j] + (float)v);
                o[j] = v;
            }
            *reinterpret_cast<h4 *>(f.out + (long)m * f.ldo + n0 + c4) = o;
        }
        return;
    }
    if (f.mode == SMH_FIN_SILU_MUL) {
        const int n_half = n_total / 2;                      // slabs hold [gate | up]
        const int g0 = cu * 256;
        for (int i = tid; i < M * 64; i += THREADS) {
            const int m = i >> 6, c4 = 4 * (i & 63);
            if (g0 + c4 >= n_half) continue;
            const f4 ga = slices_sum4(partial + (long)m * n_total + g0 + c4, slab, ksplit);
            const f4 ua = slices_sum4(partial + (long)m * n_total + n_half + g0 + c4, slab, ksplit);
            h4 o;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float gf = (float)(half_t)ga[j];
                const half_t sl = (half_t)(gf / (1.0f + expf(-gf)));
                o[j] = sl * (half_t)ua[j];
            }
            *reinterpret_cast<h4 *>(f.out + (long)m * f.ldo + g0 + c4) = o;
        }
        return;
    }
    if (f.mode == SMH_FIN_ROPE_APPEND) {
        // one wave per (row, head of the unit): lane owns the pair (d, d + 64)
        const int t = (f.t_dev != nullptr) ? *f.t_dev : -1;
        const int pos = *f.pos_dev;
        const int heads_in_unit = width / 128;
        for (int item = wave; item < M * heads_in_unit; item += WAVES) {
            const int m = item / heads_in_unit, hh = item - m * heads_in_unit;
            const int head = n_seg0 / 128 + hh;                 // head index inside its segment (q, k or v)
            const float *src = partial + (long)m * n_total + n0 + hh * 128;
            half_t x1 = (half_t)slices_sum1(src + lane, slab, ksplit);
            half_t x2 = (half_t)slices_sum1(src + 64 + lane, slab, ksplit);
            if (seg == 2) {
                half_t *pv = f.v + ((long)m * f.Hkv + head) * 128;
                pv[lane] = x1;
                pv[lane + 64] = x2;
                if (f.cache_v != nullptr && t >= 0 && t < f.Smax) {
                    const long row = ((long)m * f.Smax + t) * f.Hkv + head;
                    kv_store_row2(x1, x2, f.cache_v + row * 64, f.cache_vs + row * 2, lane);
                }
                continue;
            }
            rope_pair2(x1, x2, f.cos_tab[(long)pos * 64 + lane], f.sin_tab[(long)pos * 64 + lane]);
            if (seg == 0) {
                half_t *pq = f.q + ((long)m * f.H + head) * 128;
                pq[lane] = x1;
                pq[lane + 64] = x2;
            } else {
                half_t *pk = f.k + ((long)m * f.Hkv + head) * 128;
                pk[lane] = x1;
                pk[lane + 64] = x2;
                if (f.cache_k != nullptr && t >= 0 && t < f.Smax) {
                    const long row = ((long)m * f.Smax + t) * f.Hkv + head;
                    kv_store_row2(x1, x2, f.cache_k + row * 64, f.cache_ks + row * 2, lane);
                }
            }
        }
        return;
    }
    // ---- RESIDUAL_RMSNORM: this unit's columns of h, then (last unit only) the norm of every row ----
    for (int m = wave; m < M; m += WAVES) {
        const int c4 = 4 * lane;
        float ss = 0.f;
        if (c4 < width) {
            const f4 acc = slices_sum4(partial + (long)m * n_total + n0 + c4, slab, ksplit);
            const h4 r = *reinterpret_cast<const h4 *>(f.resid + (long)m * f.ldr + n0 + c4);
            h4 o;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const half_t v = (half_t)acc[j];
                o[j] = (half_t)((float)r[j] + (float)v);
                ss += (float)o[j] * (float)o[j];
            }
            st_h4(f.h_out + (long)m * n_total + n0 + c4, o);
        }
        ss = wave_sum(ss);
        if (lane == 0) st_f32(f.ssq + (long)unit * M + m, ss);
    }
    wait_vmem();
    __syncthreads();
    if (tid == 0) {
        const uint32_t prev = __hip_atomic_fetch_add(f.row_cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const bool last = prev == (uint32_t)units - 1u;
        if (last) st_u32(f.row_cnt, 0u);
        *s_flag = last ? 1u : 0u;
    }
    __syncthreads();
    if (*s_flag == 0u) return;
    for (int m = wave; m < M; m += WAVES) {
        float tot = 0.f;
        for (int u = lane; u < units; u += 64) tot += ld_f32(f.ssq + (long)u * M + m);
        tot = wave_sum(tot);
        const float r = rms_factor(tot, n_total, f.eps);
        for (int c4 = 4 * lane; c4 < n_total; c4 += 256) {
            const h4 hv = ld_h4(f.h_out + (long)m * n_total + c4);
            const h4 w = *reinterpret_cast<const h4 *>(f.norm_w + c4);
            h4 o;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const half_t nv = scale_to_half(hv[j], r);
                o[j] = nv * w[j];
            }
            *reinterpret_cast<h4 *>(f.xn_out + (long)m * n_total + c4) = o;
        }
    }
}

}  // namespace smh
