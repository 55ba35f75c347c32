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
    const float r = rms_factor(total, dim, eps);
    for (int i = threadIdx.x * 8; i < dim; i += 256 * 8) {
        h8 v = *reinterpret_cast<const h8 *>(xr + i);
        h8 w = *reinterpret_cast<const h8 *>(wt + i);
        h8 o;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            half_t n = scale_to_half(v[j], r);
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

namespace smh {

// ---- temperature / top-k sampling -----------------------------------------------------------------------------
// One 1024-thread workgroup per row.  x = fp16(logit / temperature) (the reference divides fp16 tensors); the k largest
// x, equal values taken lowest index first, are found with a two-pass radix select on an order-preserving 16-bit key
// (256-bin histograms in LDS), gathered, ordered by (x descending, index ascending) with a rank sort, turned into
// probabilities p = fp16(softmax) as F.softmax on an fp16 tensor returns them, and one candidate is drawn by inverse
// CDF with the caller's uniform number.
constexpr int SAMPLE_MAX_K = 1024;

__device__ __forceinline__ uint32_t sample_key(half_t x) {
    const uint32_t b = __builtin_bit_cast(uint16_t, x);
    return (b & 0x8000u) ? (~b & 0xFFFFu) : (b | 0x8000u);       // larger value <=> larger key
}
__device__ __forceinline__ half_t sample_unkey(uint32_t k) {
    const uint16_t b = (uint16_t)((k & 0x8000u) ? (k & 0x7FFFu) : (~k & 0xFFFFu));
    return __builtin_bit_cast(half_t, b);
}

// Inclusive prefix sums over the 1024 threads of the workgroup (thread order): inside a wave by lane shifts, across waves
// through s_w[16]; two barriers.  Every thread of the workgroup must call.
template <class T>
__device__ __forceinline__ T sample_block_scan(T v, T *s_w) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const T t = __shfl_up(v, o, 64);
        if (lane >= o) v += t;
    }
    if (lane == 63) s_w[wave] = v;
    __syncthreads();
    T base = 0;
    for (int w = 0; w < wave; ++w) base += s_w[w];
    __syncthreads();
    return v + base;
}

// bins[t] <- sum of bins[t..255]; then the bin where the count from the top reaches `want` and the count above it
__device__ __forceinline__ void sample_pick_bin(int *bins, int *s_w, int want, int *out_bin, int *out_above) {
    const int t = threadIdx.x;
    const int mine = t < 256 ? bins[255 - t] : 0;                 // thread t holds bin 255 - t: a prefix sum from the top
    const int upto = sample_block_scan(mine, s_w);
    if (t < 256) bins[255 - t] = upto;
    __syncthreads();
    if (t < 256) {
        const int above = t == 255 ? 0 : bins[t + 1];
        if (bins[t] >= want && above < want) { *out_bin = t; *out_above = above; }
    }
    __syncthreads();
}

// counts == nullptr: one draw per row, uniform[row] -> out[row].  Otherwise row r makes counts[r] draws with replacement from
// its candidates, with the uniform numbers (and into the slots of out) that start at counts[0] + ... + counts[r-1].
// Thread t owns the contiguous chunk of ceil(vocab / 1024) logits that starts at t times that.  Up to 32768 logits (a multiple
// of 8, rows 16-byte aligned) the chunk is read ONCE, as four 16-byte loads, and its 32 sixteen-bit keys stay in registers for
// the two histogram passes, the tie count and the gather; otherwise every pass reads the logits again.
__global__ __launch_bounds__(1024) void sample_topk_kernel(const half_t *__restrict__ logits, int vocab, long ld, float temperature,
                                                           int top_k, const float *__restrict__ uniform, int64_t *__restrict__ out,
                                                           const int32_t *__restrict__ counts, const float *__restrict__ row_temps, int n_draws,
                                                           int keep_ties) {
    // row_temps: a temperature per row, applied in fp32 (a tensor divisor promotes the fp16 logits to fp32 in torch, a
    // Python scalar does not): candidates by the raw logits (division by a positive number keeps their order, and two
    // different fp16 values stay different in fp32), softmax and probabilities in fp32
    // keep_ties: the filter form of top-k (everything below the k-th largest value is masked, so EVERY value equal to it
    // stays a candidate - up to SAMPLE_MAX_K candidates in all), on fp32 logits / temperature
    const bool wide = row_temps != nullptr || keep_ties;
    if (row_temps != nullptr) temperature = row_temps[blockIdx.x];
    // a row temperature that is not positive (a ramp that reaches 0, a NaN) has no softmax: the row draws its largest logit
    // every time (the limit of the distribution as the temperature goes to 0), lowest index first among equals
    const bool greedy_row = row_temps != nullptr && !(temperature > 0.f);
    if (greedy_row) temperature = 1.0f;
    __shared__ int bins[256];
    __shared__ int wbins[256 * 16];
    __shared__ int s_wi[16];
    __shared__ float s_wf[16];
    __shared__ int s_bin, s_above, s_count;
    __shared__ uint32_t c_key[SAMPLE_MAX_K];
    __shared__ int c_idx[SAMPLE_MAX_K];
    __shared__ uint32_t o_key[SAMPLE_MAX_K];
    __shared__ int o_idx[SAMPLE_MAX_K];
    __shared__ float cdf[SAMPLE_MAX_K];
    const int tid = threadIdx.x;
    const half_t *row = logits + (long)blockIdx.x * ld;
    int k = min(top_k, vocab);
    auto key_of = [&](half_t x) { return sample_key(wide ? x : (half_t)((float)x / temperature)); };
    auto value_of = [&](uint32_t key) { return wide ? (float)sample_unkey(key) / temperature : (float)sample_unkey(key); };

    constexpr int CH = 32;
    const bool in_regs = vocab <= 1024 * CH && vocab % 8 == 0 && (reinterpret_cast<uintptr_t>(row) & 15) == 0;     // (uniform)
    const int chunk = in_regs ? CH : (vocab + 1023) / 1024;
    const int lo = min(tid * chunk, vocab), hi = min(vocab, lo + chunk);
    uint32_t kr[CH / 2];                       // in_regs: keys of elements lo + 2 j (low half) and lo + 2 j + 1
    if (in_regs) {
        u32x4 raw[CH / 8];
#pragma unroll
        for (int q = 0; q < CH / 8; ++q) {
            raw[q] = u32x4{0u, 0u, 0u, 0u};
            if (lo + 8 * q < hi) raw[q] = *reinterpret_cast<const u32x4 *>(row + lo + 8 * q);
        }
#pragma unroll
        for (int j = 0; j < CH / 2; ++j) {
            const uint32_t two = raw[j >> 2][j & 3];
            const uint32_t k0 = key_of(__builtin_bit_cast(half_t, (uint16_t)(two & 0xFFFFu)));
            const uint32_t k1 = key_of(__builtin_bit_cast(half_t, (uint16_t)(two >> 16)));
            kr[j] = k0 | (k1 << 16);
        }
    }
    // f(index, key) for every logit of this thread's chunk, in index order
    auto for_each = [&](auto f) {
        if (in_regs) {
#pragma unroll
            for (int j = 0; j < CH; ++j)
                if (lo + j < hi) f(lo + j, (kr[j >> 1] >> (16 * (j & 1))) & 0xFFFFu);
        } else {
            for (int i = lo; i < hi; ++i) f(i, key_of(row[i]));
        }
    };

    // ---- the k-th largest key: high byte, then low byte ----
    // Atomics of different waves on one LDS word take turns, and logits crowd into a few high bytes: every wave counts into a
    // histogram of its own (word = bin * 16 + wave, the 16 copies of a bin in 16 banks), which are then added.
    const int wv = tid >> 6;
    auto fold_bins = [&]() {
        if (tid < 256) {
            int n = 0;
#pragma unroll
            for (int w = 0; w < 16; ++w) n += wbins[tid * 16 + w];
            bins[tid] = n;
        }
        __syncthreads();
    };
    for (int i = tid; i < 256 * 16; i += 1024) wbins[i] = 0;
    if (tid == 0) s_count = 0;
    __syncthreads();
    for_each([&](int, uint32_t key) { atomicAdd(&wbins[(key >> 8) * 16 + wv], 1); });
    __syncthreads();
    fold_bins();
    sample_pick_bin(bins, s_wi, k, &s_bin, &s_above);
    const int b1 = s_bin, above1 = s_above;
    __syncthreads();
    for (int i = tid; i < 256 * 16; i += 1024) wbins[i] = 0;
    __syncthreads();
    for_each([&](int, uint32_t key) {
        if ((int)(key >> 8) == b1) atomicAdd(&wbins[(key & 255u) * 16 + wv], 1);
    });
    __syncthreads();
    fold_bins();
    sample_pick_bin(bins, s_wi, k - above1, &s_bin, &s_above);
    const uint32_t kth = ((uint32_t)b1 << 8) | (uint32_t)s_bin;      // key of the k-th largest value
    int ties_wanted = k - (above1 + s_above);                          // how many of the values equal to it are in
    if (keep_ties) {                                                   // all of them, while the candidate arrays hold them
        ties_wanted = min(bins[s_bin] - s_above, SAMPLE_MAX_K - (above1 + s_above));
        k = above1 + s_above + ties_wanted;
    }
    __syncthreads();

    // ---- gather: everything above the k-th key, and of the ties the lowest indices (the chunks are in index order, so a
    //      prefix sum of the per-thread tie counts gives each tie its rank by index) ----
    int my_ties = 0;
    for_each([&](int, uint32_t key) { my_ties += key == kth; });
    int tie_rank = sample_block_scan(my_ties, s_wi) - my_ties;         // ties at lower indices
    for_each([&](int i, uint32_t key) {
        bool take = key > kth;
        if (key == kth) { take = tie_rank < ties_wanted; ++tie_rank; }
        if (take) {
            const int slot = atomicAdd(&s_count, 1);
            c_key[slot] = key;
            c_idx[slot] = i;
        }
    });
    __syncthreads();

    // ---- order the k candidates: rank = number of candidates that come before ----
    if (tid < k) {
        const uint32_t mk = c_key[tid];
        const int mi = c_idx[tid];
        int rank = 0;
        for (int j = 0; j < k; ++j) rank += (c_key[j] > mk) || (c_key[j] == mk && c_idx[j] < mi);
        o_key[rank] = mk;
        o_idx[rank] = mi;
    }
    __syncthreads();

    // ---- p = fp16(softmax) (fp32 with a row temperature or the filter form), inverse CDF ----
    const float xmax = value_of(o_key[0]);
    const float e = tid < k ? expf(value_of(o_key[tid]) - xmax) : 0.f;
    cdf[tid] = sample_block_scan(e, s_wf);
    __syncthreads();
    const float total = cdf[k - 1];
    __syncthreads();
    const float pr = tid < k ? (wide ? e / total : (float)(half_t)(e / total)) : 0.f;
    cdf[tid] = sample_block_scan(pr, s_wf);
    __syncthreads();
    long first = blockIdx.x;
    int draws = 1;
    if (counts != nullptr) {
        first = 0;
        for (int r = 0; r < (int)blockIdx.x; ++r) first += max(counts[r], 0);
        draws = max(counts[blockIdx.x], 0);
        draws = (int)max(min((long)draws, (long)n_draws - first), 0L);       // counts that add up to more than the buffers hold are cut
    }
    if (greedy_row) {
        for (int j = tid; j < draws; j += 1024) out[first + j] = o_idx[0];
        return;
    }
    if (tid < k) {
        const float before = tid == 0 ? 0.f : cdf[tid - 1];
        for (int j = 0; j < draws; ++j) {
            const float target = uniform[first + j] * cdf[k - 1];
            // first candidate whose cumulative probability exceeds the target (the last one if rounding leaves none)
            if ((before <= target && target < cdf[tid]) || (tid == k - 1 && target >= cdf[tid])) out[first + j] = o_idx[tid];
        }
    }
}

// The bookkeeping of one step of the tree sampler (mcts.py:127-152) for all branches in one launch, one workgroup.
//   draws   the tokens every live branch drew this step (sample_topk_kernel with counts): branch i owns cnt[i] of them,
//           in branch order
//   per branch i < *curr_b, in order: its distinct tokens in ascending order with their multiplicities (torch.unique,
//           :131); if the branch is alive the smallest stays on row i with its multiplicity (:135-138) and each further
//           distinct token opens a new row while rows are left (:141-150): the new row takes the origin's token
//           history, the token, its multiplicity, and - instead of a copy of K/V rows - the origin's page ids of the
//           suffix rows written so far.  Dead branches change nothing.  Then the step's column of every dead row is
//           zeroed (:160).
//   tok / cnt = output_counts[0] / [1] of the reference; origin[r] = the branch row r was forked from in this step, else -1.
constexpr int TREE_MAX_BATCH = 1024;
// What follows the fork in a step of the search loop (mcts.py:160-175), for the variant that does the whole step in one launch:
// the terminal state machine on the step's column, the lengths and the mask of live rows, the tokens the next forward
// reads, and the two numbers the host needs (branches, ended rows).
struct TreeFinish {
    int32_t *state;              // end_stateMachine [batch_size]
    const int64_t *seq;          // the terminal sequence
    int seq_len;
    int64_t eos;
    int32_t *results_len;        // [batch_size]
    int64_t *next_tokens;        // [batch_size]: column t of results, the next decode step's input
    int32_t *summary;            // [2]: branches after the step, rows that have ended
};
// t_dev != nullptr: the step's column AND the suffix rows written so far are *t_dev (a search step t follows t decode steps),
// read on the device so that one captured launch serves every step.
__global__ __launch_bounds__(256) void tree_fork_kernel(const int64_t *__restrict__ draws, int n_draws, int32_t *__restrict__ tok, int32_t *__restrict__ cnt,
                                                        uint8_t *__restrict__ alive, int32_t *__restrict__ curr_b, int batch_size,
                                                        int64_t *__restrict__ results, long ld, int t,
                                                        int32_t *__restrict__ pages, long pages_stride, int n_rows,
                                                        int32_t *__restrict__ origin, const int32_t *__restrict__ t_dev, TreeFinish fin) {
    if (t_dev != nullptr) {
        t = min(max(*t_dev, 0), (int)ld - 1);                    // (a counter outside the row is cut, never followed)
        n_rows = (int)min((long)t, pages_stride);
    }
    __shared__ uint64_t keys[TREE_MAX_BATCH];      // (branch, token) of every draw, sorted by the whole workgroup
    __shared__ int64_t u_tok[TREE_MAX_BATCH];      // per branch its distinct tokens in ascending order (at the segment's start)
    __shared__ int u_cnt[TREE_MAX_BATCH];          // ... and their multiplicities
    __shared__ int seg_off[TREE_MAX_BATCH + 1];    // first draw of branch i
    __shared__ int seg_uniq[TREE_MAX_BATCH];       // distinct tokens of branch i
    __shared__ int scan[TREE_MAX_BATCH + 1];       // distinct (branch, token) pairs before position i
    __shared__ int start[TREE_MAX_BATCH + 1];      // first position of the u-th distinct pair
    __shared__ int wave_sum[4];
    __shared__ int s_new;                          // branches after the step
    const int tid = threadIdx.x;
    const int c0 = min(max(*curr_b, 0), batch_size);             // (a counter outside the batch is cut, never followed)
    if (tid == 0) {
        int off = 0;
        for (int i = 0; i < c0; ++i) { seg_off[i] = off; off = min(off + max(cnt[i], 0), TREE_MAX_BATCH); }
        seg_off[c0] = off;
    }
    __syncthreads();
    const int total = min(seg_off[c0], min(n_draws, TREE_MAX_BATCH));   // draws the buffer does not hold do not exist
    // key of draw i: its branch (the last one whose segment starts at or before i, found by bisection) above its token;
    // slots past the draws sort to the end
    for (int i = tid; i < TREE_MAX_BATCH; i += 256) {
        uint64_t key = ~0ull;
        if (i < total) {
            int lo = 0, hi = c0 - 1;
            while (lo < hi) {
                const int mid = (lo + hi + 1) >> 1;
                if (seg_off[mid] <= i) lo = mid; else hi = mid - 1;
            }
            key = ((uint64_t)(uint32_t)lo << 32) | (uint64_t)(uint32_t)draws[i];
        }
        keys[i] = key;
    }
    for (int r = tid; r < batch_size; r += 256) origin[r] = -1;
    __syncthreads();
    // bitonic sort of the keys by the whole workgroup, over the smallest power of two that holds the draws (the slots
    // past them hold the largest key and stay behind)
    int n_sort = 2;
    while (n_sort < total) n_sort <<= 1;
    for (int k = 2; k <= n_sort; k <<= 1)
        for (int j = k >> 1; j > 0; j >>= 1) {
            for (int x = tid; x < n_sort / 2; x += 256) {
                const int i = ((x & ~(j - 1)) << 1) | (x & (j - 1));        // the lower index of the pair (i, i + j)
                const uint64_t a = keys[i], b = keys[i + j];
                const bool up = (i & k) == 0;
                if ((a > b) == up) { keys[i] = b; keys[i + j] = a; }
            }
            __syncthreads();
        }
    // run-length encoding by the whole workgroup: a position opens a run when its key differs from its predecessor's
    // (a new branch always does); an exclusive scan numbers the runs, start[u] is where run u begins
    {
        int head[4], local = 0;
        const int base = tid * 4;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int i = base + e;
            head[e] = (i < total && (i == 0 || keys[i] != keys[i - 1])) ? 1 : 0;
            local += head[e];
        }
        int incl = local;                                   // inclusive scan over the 256 threads: wave scan, then wave sums
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int v = __shfl_up(incl, o, 64);
            if ((tid & 63) >= o) incl += v;
        }
        if ((tid & 63) == 63) wave_sum[tid >> 6] = incl;
        __syncthreads();
        int before = incl - local;
        for (int w = 0; w < (tid >> 6); ++w) before += wave_sum[w];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            scan[base + e] = before;
            if (head[e]) start[before] = base + e;
            before += head[e];
        }
        if (tid == 255) { scan[TREE_MAX_BATCH] = before; start[before] = total; }
    }
    __syncthreads();
    const int n_runs = scan[TREE_MAX_BATCH];
    for (int i = tid; i < c0; i += 256) {
        const int lo = min(seg_off[i], total), hi = min(seg_off[i + 1], total);
        seg_uniq[i] = scan[hi] - scan[lo];                  // (scan[total] counts every run: no run opens past the draws)
    }
    for (int u = tid; u < n_runs; u += 256) {
        const int at = start[u];
        const int br = (int)(keys[at] >> 32);
        const int slot = min(seg_off[br], total) + (u - scan[min(seg_off[br], total)]);
        u_tok[slot] = (int64_t)(int32_t)(uint32_t)keys[at];
        u_cnt[slot] = start[u + 1] - at;
    }
    __syncthreads();
    // rows are handed out in branch order (what is left depends on every earlier branch): one thread walks the branches
    if (tid == 0) {
        int cur = c0;
        for (int i = 0; i < c0; ++i) {
            if (!alive[i] || seg_uniq[i] == 0) continue;
            const int lo = seg_off[i];
            tok[i] = (int32_t)u_tok[lo];
            cnt[i] = u_cnt[lo];
            const int forks = min(seg_uniq[i] - 1, batch_size - cur);
            for (int j = 0; j < forks; ++j) {
                origin[cur + j] = i;
                tok[cur + j] = (int32_t)u_tok[lo + 1 + j];
                cnt[cur + j] = u_cnt[lo + 1 + j];
            }
            cur += max(forks, 0);
        }
        s_new = cur;
        *curr_b = cur;
    }
    __syncthreads();
    const int c1 = s_new;
    // token histories and page ids of the new rows, then this step's column
    for (int r = c0; r < c1; ++r) {
        const int o = origin[r];
        for (long j = tid; j < ld; j += 256) results[(long)r * ld + j] = results[(long)o * ld + j];
        if (pages != nullptr)
            for (int j = tid; j < n_rows; j += 256) pages[(long)r * pages_stride + j] = pages[(long)o * pages_stride + j];
    }
    __syncthreads();
    int ended = 0;
    for (int r = tid; r < batch_size; r += 256) {
        int64_t token = results[(long)r * ld + t];
        if (!alive[r]) token = 0;
        else if (r < c1 && (r >= c0 || seg_uniq[r] > 0)) token = tok[r];
        results[(long)r * ld + t] = token;
        if (fin.state != nullptr) {
            // detectTerminal on the step's column (mcts.py:14-28, :162), lengths and mask (:163-164)
            const int32_t st = fin.state[r];
            const int32_t match = (st >= 0 && st < fin.seq_len && fin.seq[st] == token) ? 1 : 0;
            const int32_t nxt = (st + match) * match;
            const bool done = nxt == fin.seq_len || token == fin.eos;
            fin.state[r] = done ? 0 : nxt;
            const bool was = alive[r] != 0;
            fin.results_len[r] += was ? 1 : 0;
            const bool now = was && !done;
            alive[r] = now ? 1 : 0;
            ended += now ? 0 : 1;
            fin.next_tokens[r] = token;
        }
    }
    if (fin.state != nullptr) {
        __syncthreads();                            // (scan[] is free again)
        scan[tid] = ended;
        __syncthreads();
        for (int o = 128; o > 0; o >>= 1) {
            if (tid < o) scan[tid] += scan[tid + o];
            __syncthreads();
        }
        if (tid == 0) { fin.summary[0] = c1; fin.summary[1] = scan[0]; }
    }
}

}  // namespace smh

extern "C" int smh_sample_topk(const void *logits, int rows, int vocab, long ld, float temperature, int top_k,
                               const float *uniform, int64_t *out, smh_stream_t stream) {
    using namespace smh;
    SMH_REQUIRE(rows >= 0 && vocab > 0 && ld >= vocab, "smh_sample_topk: rows=%d vocab=%d ld=%ld", rows, vocab, ld);
    SMH_REQUIRE(top_k >= 1 && top_k <= SAMPLE_MAX_K, "smh_sample_topk: top_k=%d outside [1,%d]", top_k, SAMPLE_MAX_K);
    SMH_REQUIRE(temperature > 0.f, "smh_sample_topk: temperature=%g must be positive (greedy decoding is smh_argmax)", (double)temperature);
    if (rows == 0) return 0;
    SMH_REQUIRE(logits && uniform && out, "smh_sample_topk: null pointer");
    hipLaunchKernelGGL(sample_topk_kernel, dim3(rows), dim3(1024), 0, (hipStream_t)stream, (const half_t *)logits, vocab, ld, temperature,
                       top_k, uniform, out, (const int32_t *)nullptr, (const float *)nullptr, rows, 0);
    return launch_status();
}

extern "C" int smh_sample_topk_filter(const void *logits, int rows, int vocab, long ld, float temperature, int top_k,
                                      const float *uniform, int64_t *out, smh_stream_t stream) {
    using namespace smh;
    SMH_REQUIRE(rows >= 0 && vocab > 0 && ld >= vocab, "smh_sample_topk_filter: rows=%d vocab=%d ld=%ld", rows, vocab, ld);
    SMH_REQUIRE(top_k >= 1 && top_k <= SAMPLE_MAX_K, "smh_sample_topk_filter: top_k=%d outside [1,%d]", top_k, SAMPLE_MAX_K);
    SMH_REQUIRE(temperature > 0.f, "smh_sample_topk_filter: temperature=%g must be positive (greedy decoding is smh_argmax)", (double)temperature);
    if (rows == 0) return 0;
    SMH_REQUIRE(logits && uniform && out, "smh_sample_topk_filter: null pointer");
    hipLaunchKernelGGL(sample_topk_kernel, dim3(rows), dim3(1024), 0, (hipStream_t)stream, (const half_t *)logits, vocab, ld, temperature,
                       top_k, uniform, out, (const int32_t *)nullptr, (const float *)nullptr, rows, 1);
    return launch_status();
}

extern "C" int smh_sample_topk_counts(const void *logits, int rows, int vocab, long ld, float temperature, int top_k,
                                      const float *uniform, const int32_t *counts, int64_t *out, int n_draws, smh_stream_t stream) {
    using namespace smh;
    SMH_REQUIRE(rows >= 0 && rows <= TREE_MAX_BATCH && vocab > 0 && ld >= vocab, "smh_sample_topk_counts: rows=%d (at most %d) vocab=%d ld=%ld", rows, TREE_MAX_BATCH, vocab, ld);
    SMH_REQUIRE(top_k >= 1 && top_k <= SAMPLE_MAX_K, "smh_sample_topk_counts: top_k=%d outside [1,%d]", top_k, SAMPLE_MAX_K);
    SMH_REQUIRE(temperature > 0.f, "smh_sample_topk_counts: temperature=%g must be positive", (double)temperature);
    if (rows == 0) return 0;
    SMH_REQUIRE(logits && uniform && counts && out && n_draws >= 0, "smh_sample_topk_counts: null pointer or n_draws=%d", n_draws);
    hipLaunchKernelGGL(sample_topk_kernel, dim3(rows), dim3(1024), 0, (hipStream_t)stream, (const half_t *)logits, vocab, ld, temperature,
                       top_k, uniform, out, counts, (const float *)nullptr, n_draws, 0);
    return launch_status();
}

extern "C" int smh_sample_topk_rowtemp(const void *logits, int rows, int vocab, long ld, const float *row_temps, int top_k,
                                       const float *uniform, const int32_t *counts, int64_t *out, int n_draws, smh_stream_t stream) {
    using namespace smh;
    SMH_REQUIRE(rows >= 0 && rows <= TREE_MAX_BATCH && vocab > 0 && ld >= vocab, "smh_sample_topk_rowtemp: rows=%d (at most %d) vocab=%d ld=%ld", rows, TREE_MAX_BATCH, vocab, ld);
    SMH_REQUIRE(top_k >= 1 && top_k <= SAMPLE_MAX_K, "smh_sample_topk_rowtemp: top_k=%d outside [1,%d]", top_k, SAMPLE_MAX_K);
    if (rows == 0) return 0;
    SMH_REQUIRE(logits && row_temps && uniform && counts && out && n_draws >= 0, "smh_sample_topk_rowtemp: null pointer or n_draws=%d", n_draws);
    hipLaunchKernelGGL(sample_topk_kernel, dim3(rows), dim3(1024), 0, (hipStream_t)stream, (const half_t *)logits, vocab, ld, 1.0f,
                       top_k, uniform, out, counts, row_temps, n_draws, 0);
    return launch_status();
}

extern "C" int smh_tree_fork(const int64_t *draws, int n_draws, int32_t *tok, int32_t *cnt, const uint8_t *alive, int32_t *curr_b, int batch_size,
                             int64_t *results, long ld, int t, int32_t *pages, long pages_stride, int n_rows, int32_t *origin,
                             smh_stream_t stream) {
    using namespace smh;
    SMH_REQUIRE(batch_size >= 1 && batch_size <= TREE_MAX_BATCH, "smh_tree_fork: batch_size=%d outside [1,%d]", batch_size, TREE_MAX_BATCH);
    SMH_REQUIRE(draws && n_draws >= 0 && tok && cnt && alive && curr_b && results && origin, "smh_tree_fork: null pointer or n_draws=%d", n_draws);
    SMH_REQUIRE(ld >= 1 && t >= 0 && t < ld, "smh_tree_fork: column %d outside the %ld of a row", t, ld);
    SMH_REQUIRE(pages == nullptr || (pages_stride >= n_rows && n_rows >= 0), "smh_tree_fork: n_rows=%d pages_stride=%ld", n_rows, pages_stride);
    hipLaunchKernelGGL(tree_fork_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, draws, n_draws, tok, cnt, const_cast<uint8_t *>(alive), curr_b, batch_size,
                       results, ld, t, pages, pages_stride, n_rows, origin, (const int32_t *)nullptr, TreeFinish{});
    return launch_status();
}

extern "C" int smh_tree_step(const int64_t *draws, int n_draws, int32_t *tok, int32_t *cnt, uint8_t *alive, int32_t *curr_b, int batch_size,
                             int64_t *results, long ld, const int32_t *t_dev, int32_t *pages, long pages_stride, int32_t *origin,
                             int32_t *state, const int64_t *terminal_seq, int seq_len, int64_t eos, int32_t *results_len,
                             int64_t *next_tokens, int32_t *summary, smh_stream_t stream) {
    using namespace smh;
    SMH_REQUIRE(batch_size >= 1 && batch_size <= TREE_MAX_BATCH, "smh_tree_step: batch_size=%d outside [1,%d]", batch_size, TREE_MAX_BATCH);
    SMH_REQUIRE(draws && n_draws >= 0 && tok && cnt && alive && curr_b && results && origin && t_dev, "smh_tree_step: null pointer or n_draws=%d", n_draws);
    SMH_REQUIRE(ld >= 1 && (pages == nullptr || pages_stride >= 1), "smh_tree_step: ld=%ld pages_stride=%ld", ld, pages_stride);
    SMH_REQUIRE(state && terminal_seq && seq_len >= 1 && results_len && next_tokens && summary, "smh_tree_step: null pointer or seq_len=%d", seq_len);
    TreeFinish fin{state, terminal_seq, seq_len, eos, results_len, next_tokens, summary};
    hipLaunchKernelGGL(tree_fork_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, draws, n_draws, tok, cnt, alive, curr_b, batch_size, results, ld, 0,
                       pages, pages_stride, 0, origin, t_dev, fin);
    return launch_status();
}

namespace smh {

// detectTerminal of the tree sampler (mcts.py:14-28), one thread per branch: the state counts how many tokens of the
// terminal sequence the branch has produced in a row; a token that does not continue it sends the state back to 0
// (also when it equals the sequence's first token, as in the reference); the branch ends when the sequence is
// complete or the token is the end-of-sequence id, and an ended branch restarts at state 0.
__global__ __launch_bounds__(256) void detect_terminal_kernel(const int64_t *__restrict__ token, int32_t *__restrict__ state,
                                                             uint8_t *__restrict__ end, const int64_t *__restrict__ seq, int seq_len,
                                                             int64_t eos, int rows) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= rows) return;
    const int64_t tok = token[i];
    const int32_t st = state[i];
    const int32_t match = (st >= 0 && st < seq_len && seq[st] == tok) ? 1 : 0;
    int32_t nxt = (st + match) * match;
    const bool done = nxt == seq_len || tok == eos;
    end[i] = done ? 1 : 0;
    state[i] = done ? 0 : nxt;
}

}  // namespace smh

extern "C" int smh_detect_terminal(const int64_t *token, int32_t *state, uint8_t *end, const int64_t *terminal_seq, int seq_len,
                                   int64_t eos, int rows, smh_stream_t stream) {
    using namespace smh;
    SMH_REQUIRE(rows >= 0 && seq_len >= 1, "smh_detect_terminal: rows=%d seq_len=%d", rows, seq_len);
    if (rows == 0) return 0;
    SMH_REQUIRE(token && state && end && terminal_seq, "smh_detect_terminal: null pointer");
    hipLaunchKernelGGL(detect_terminal_kernel, dim3((rows + 255) / 256), dim3(256), 0, (hipStream_t)stream, token, state, end,
                       terminal_seq, seq_len, eos, rows);
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

namespace smh {
__global__ void set_step_kernel(int32_t *state, int pos, int t) {
    state[0] = pos;
    state[1] = t;
}
}  // namespace smh

extern "C" int smh_set_step(int32_t *state, int pos, int t, smh_stream_t stream) {
    SMH_REQUIRE(state != nullptr && pos >= 0 && t >= 0, "smh_set_step: state=%p pos=%d t=%d", (void *)state, pos, t);
    hipLaunchKernelGGL(smh::set_step_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, state, pos, t);
    return smh::launch_status();
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
