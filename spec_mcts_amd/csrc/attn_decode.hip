// Shared-prefix decode attention: one query per (branch, head) over
//   [ prefix K/V (P rows, fp16, shared by all branches) || that branch's suffix (fp16 or Q4_0 rows)
//     || the new token's exact fp16 K/V ].
//
// Two kernels.
//  1. attn_prefix_kernel, grid (splits, kv heads, query groups): a workgroup stages one slice of the
//     prefix for one kv head in LDS ONCE (K row-major, V transposed) and the branches' queries for
//     that head are multiplied against it on the matrix cores: the queries are the N dimension of
//     S^T = K . Q^T and of O^T = V^T . P^T, so the prefix is read from HBM once per head instead of
//     once per branch (with many queries a slice's query tiles are dealt to a few workgroups, which
//     re-read it from the cache).  Each (slice, query) leaves an un-normalised partial (max, sum, o[128]).
//  2. attn_suffix_kernel, one wave per (branch, query head): streams the branch's own suffix rows
//     (HBM-bound; Q4_0 rows are decoded in registers), keeps an online softmax per 16-lane group,
//     folds in the prefix partials and the new token, normalises and writes fp16.
// Scores and softmax are fp32 throughout (exp2 of log2(e)-scaled scores); probabilities are rounded
// to fp16 only as the operand of the P.V matrix product.
//
// Algorithmic HBM traffic: prefix 2*P*Hkv*D*2 B once + per branch its suffix rows
// (512 B fp16 or 136 B Q4_0 per row and kv head) + q/out.
#include <mutex>

#include "attn_rows.hpp"
#include "rope_kv.hpp"

namespace smh {

constexpr int ATT_D = 128;
constexpr int ATT_TW_MAX = 128;            // prefix rows per workgroup
constexpr int ATT_KPITCH = 136;            // halves per LDS row of K (272 B: 16 rows hit distinct banks)
constexpr float LOG2E = 1.4426950408889634f;
constexpr int ATT_ONE_TW = 64;             // prefix rows per workgroup of the one-launch kernel: two workgroups fit a compute unit
constexpr int ATT_FUSED_MAX_Q = 128;       // queries per kv head (branches x query heads per kv head) of the fused variant

struct AttnParams {
    const half_t *q;
    half_t *out;
    const half_t *prefix_k, *prefix_v;
    const void *suffix_k, *suffix_v;
    const half_t *suffix_ks, *suffix_vs;
    const int32_t *lens;
    const half_t *cur_k, *cur_v;
    float *part_o;           // [splits][Hkv][Bq][128]
    float *part_ml;          // [splits][Hkv][Bq][2]
    long suffix_batch_stride_rows;   // rows (tokens) between consecutive branches of the suffix
    // paged suffix: row j of branch b is pool row pages[b * pages_stride + j] instead of b * suffix_batch_stride_rows + j
    // (page ids of page_bytes = 2, 4 or 8 bytes each); pages == nullptr: contiguous rows per branch
    const void *pages;
    long pages_stride;
    int page_bytes;
    long pool_rows;          // rows of the pool the page ids point into: an id outside 0 .. pool_rows-1 reads the nearest row, never past the pool
    // element strides of the fp16 K/V tensors: between consecutive rows (tokens) and between kv heads.  Token-major
    // [rows, Hkv, 128] is (Hkv * 128, 128); a head-major pool [Hkv, rows, 128] is (128, rows * 128).  Q4_0 rows are token-major.
    long pfx_row_stride, pfx_head_stride;
    long sfx_row_stride, sfx_head_stride;
    int B, H, Hkv, n_rep, Bq;        // Bq = B * n_rep queries per kv head
    int suffix_waves;                // waves that share one query's suffix rows (1, 2 or 4)
    int P, tw, splits;
    int suffix_format, lens_stride;
    int causal;                      // prefill mode: branch b attends to suffix rows 0..b
    float scale_log2;                // log2(e) / sqrt(D)
    // FUSED kernels: q, the new token's k and v come straight from the fp32 K-slice slabs of the wq|wk|wv product
    // ([qkv_ks][B][(H + 2 Hkv) * 128]); RoPE, the fp16 rounding points and the Q4_0 append of k, v are those of
    // partial_rope_append_kernel (q / cur_k / cur_v above are not read)
    const float *qkv;
    int qkv_ks;
    const half_t *cos_tab, *sin_tab;
    const int32_t *pos_dev;
    uint8_t *app_k, *app_v;          // the branches' suffix caches (row *app_t of every branch is written); may be null
    half_t *app_ks, *app_vs;
    const int32_t *app_t;
    int app_smax;
    uint32_t *counters;              // one-launch variant: arrivals per kv head (zero between launches)
};

// x / n_rep and x % n_rep for the query heads per kv head; 1 (multi-head attention) needs no division
__device__ __forceinline__ int div_rep(const AttnParams &p, int x) { return p.n_rep == 1 ? x : x / p.n_rep; }
__device__ __forceinline__ int mod_rep(const AttnParams &p, int x) { return p.n_rep == 1 ? 0 : x % p.n_rep; }

// column `col` of branch b in the fused q|k|v product: the slabs added in slice order, rounded once to fp16
__device__ __forceinline__ half_t qkv_value(const AttnParams &p, int b, int col) {
    const int cols = (p.H + 2 * p.Hkv) * ATT_D;
    const float *src = p.qkv + (long)b * cols + col;
    const long slab = (long)p.B * cols;
    float v[16];
#pragma unroll
    for (int s_ = 0; s_ < 16; ++s_) v[s_] = (s_ < p.qkv_ks) ? src[s_ * slab] : 0.f;
    float tot = 0.f;
#pragma unroll
    for (int s_ = 0; s_ < 16; ++s_) tot += v[s_];
    return (half_t)tot;
}
// the same in two steps, so that a caller can request several columns before it waits for any of them
struct SlabColumn { float v[16]; };
__device__ __forceinline__ void qkv_request(const AttnParams &p, int b, int col, SlabColumn &c) {
    const int cols = (p.H + 2 * p.Hkv) * ATT_D;
    const float *src = p.qkv + (long)b * cols + col;
    const long slab = (long)p.B * cols;
#pragma unroll
    for (int s_ = 0; s_ < 16; ++s_) c.v[s_] = (s_ < p.qkv_ks) ? src[s_ * slab] : 0.f;
}
__device__ __forceinline__ half_t qkv_sum(const SlabColumn &c) {
    float tot = 0.f;
#pragma unroll
    for (int s_ = 0; s_ < 16; ++s_) tot += c.v[s_];
    return (half_t)tot;
}
// four consecutive columns (col % 4 == 0)
__device__ __forceinline__ h4 qkv_value4(const AttnParams &p, int b, int col) {
    const int cols = (p.H + 2 * p.Hkv) * ATT_D;
    const float *src = p.qkv + (long)b * cols + col;
    const long slab = (long)p.B * cols;
    f4 v[16];
#pragma unroll
    for (int s_ = 0; s_ < 16; ++s_) v[s_] = (s_ < p.qkv_ks) ? *reinterpret_cast<const f4 *>(src + s_ * slab) : f4{0.f, 0.f, 0.f, 0.f};
    f4 tot = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s_ = 0; s_ < 16; ++s_) tot += v[s_];
    return h4{(half_t)tot[0], (half_t)tot[1], (half_t)tot[2], (half_t)tot[3]};
}

// position of prefix row t (0..tw-1) inside an LDS row of V^T: within each block of 32 rows the
// order is chosen so that the 8 probabilities a lane holds after two S^T tiles (rows 4g+r of tile 2j
// and of tile 2j+1) are 8 consecutive halves.
// dims 4cc..4cc+3 (lo) and 64+4cc.. (hi) of the rotated query of head h, branch b: the rotation pairs d and d + 64
// sit in the same lane
__device__ __forceinline__ void qkv_query(const AttnParams &p, int b, int h, int pos, int cc, h4 &lo, h4 &hi) {
    lo = qkv_value4(p, b, h * ATT_D + 4 * cc);
    hi = qkv_value4(p, b, h * ATT_D + 64 + 4 * cc);
    const h4 cs = *reinterpret_cast<const h4 *>(p.cos_tab + (long)pos * 64 + 4 * cc);
    const h4 sn = *reinterpret_cast<const h4 *>(p.sin_tab + (long)pos * 64 + 4 * cc);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        half_t x1 = lo[j], x2 = hi[j];
        rope_pair2(x1, x2, cs[j], sn[j]);
        lo[j] = x1; hi[j] = x2;
    }
}

__device__ __forceinline__ int vt_pos(int t) {
    const int blk = t & ~31, w = t & 31;
    const int j2 = w >> 4, g = (w >> 2) & 3, r = w & 3;
    return blk + 8 * g + 4 * j2 + r;
}

// COHERENT: the partials are read by another workgroup of the same launch (device-scope stores)
// TWM: most prefix rows a workgroup takes (p.tw <= TWM), which sizes its LDS
// qg, n_qg: this workgroup takes the query tiles of rounds qg, qg + n_qg, ... (a round = one tile per wave)
template <bool FUSED, bool COHERENT, int TWM>
__device__ __forceinline__ void attn_prefix_body(const AttnParams &p, int split, int hk, int qg = 0, int n_qg = 1) {
    __shared__ __attribute__((aligned(16))) half_t ks[TWM][ATT_KPITCH];
    __shared__ __attribute__((aligned(16))) half_t vt[ATT_D][TWM + 8];
    __shared__ __attribute__((aligned(16))) half_t qs[FUSED ? ATT_FUSED_MAX_Q : 1][ATT_D + 8];      // FUSED: the rotated queries of this kv head

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63, c = lane & 15, g = lane >> 4;
    const int t0 = split * p.tw;
    const int cnt = min(p.tw, p.P - t0);
    const int tw32 = (cnt + 31) & ~31;          // rows actually touched by the matrix ops

    // the B operand of S^T = K . Q^T for query tile qt: dims 32*k4 + 8g .. +7 of query row c
    const int q_tiles = (p.Bq + 15) / 16;
    auto load_q = [&](int qt, h8 (&qb)[4]) {
        const int qr = min(qt * 16 + c, p.Bq - 1);
        if (!FUSED) {
            const int b = div_rep(p, qr), r_ = mod_rep(p, qr);
            const half_t *qp = p.q + ((long)b * p.H + hk * p.n_rep + r_) * ATT_D + 8 * g;
#pragma unroll
            for (int k4 = 0; k4 < 4; ++k4) qb[k4] = *reinterpret_cast<const h8 *>(qp + 32 * k4);
        } else {
#pragma unroll
            for (int k4 = 0; k4 < 4; ++k4) qb[k4] = *reinterpret_cast<const h8 *>(&qs[qr][32 * k4 + 8 * g]);
        }
    };
    // un-fused: the first tile's query is requested before the prefix slice is staged
    h8 qb_first[4];
    const int qt_first = wave + 4 * qg;
    if (!FUSED && qt_first < q_tiles) load_q(qt_first, qb_first);

    // ---- stage K (row-major) and V (transposed) ----
    // A thread moves piece ch (8 dims) of FOUR consecutive rows 4 kg .. 4 kg + 3: their V values sit side by side in a
    // row of vt (vt_pos), so V goes out as 8-byte stores instead of 2-byte ones.
    const int ch = tid & 15;
    auto stage_load4 = [&](int kg, u32x4 (&kv)[4], u32x4 (&vv)[4]) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int t = 4 * kg + e;
            kv[e] = u32x4{0, 0, 0, 0}; vv[e] = u32x4{0, 0, 0, 0};
            if (t < cnt) {
                const long off = (long)(t0 + t) * p.pfx_row_stride + (long)hk * p.pfx_head_stride + ch * 8;
                kv[e] = *reinterpret_cast<const u32x4 *>(p.prefix_k + off);
                vv[e] = *reinterpret_cast<const u32x4 *>(p.prefix_v + off);
            }
        }
    };
    auto stage_store4 = [&](int kg, const u32x4 (&kv)[4], const u32x4 (&vv)[4]) {
#pragma unroll
        for (int e = 0; e < 4; ++e) *reinterpret_cast<u32x4 *>(&ks[4 * kg + e][ch * 8]) = kv[e];
        const int pos = vt_pos(4 * kg);
        const h8 v0 = __builtin_bit_cast(h8, vv[0]), v1 = __builtin_bit_cast(h8, vv[1]);
        const h8 v2 = __builtin_bit_cast(h8, vv[2]), v3 = __builtin_bit_cast(h8, vv[3]);
#pragma unroll
        for (int j = 0; j < 8; ++j) *reinterpret_cast<h4 *>(&vt[ch * 8 + j][pos]) = h4{v0[j], v1[j], v2[j], v3[j]};
    };
    auto build_queries = [&]() {
        const int cc = tid & 15;
        const int pos = *p.pos_dev;
        for (int qr = tid >> 4; qr < p.Bq; qr += 16) {
            h4 lo, hi;
            qkv_query(p, div_rep(p, qr), hk * p.n_rep + mod_rep(p, qr), pos, cc, lo, hi);
            *reinterpret_cast<h4 *>(&qs[qr][4 * cc]) = lo;
            *reinterpret_cast<h4 *>(&qs[qr][64 + 4 * cc]) = hi;
        }
    };
    if (FUSED && TWM <= 64) {
        // every load of the workgroup is requested before anything waits: the K / V slice into registers, then
        // the slabs from which all 256 threads build the rotated queries of this kv head (8 dims each)
        static_assert(!FUSED || TWM > 64 || TWM == 64, "one group of four rows per thread");
        u32x4 kv[4], vv[4];
        const int kg = tid >> 4;
        if (4 * kg < tw32) stage_load4(kg, kv, vv);
        build_queries();
        if (4 * kg < tw32) stage_store4(kg, kv, vv);
    } else {
        if (FUSED) build_queries();
        for (int kg = tid >> 4; 4 * kg < tw32; kg += 16) {
            u32x4 kv[4], vv[4];
            stage_load4(kg, kv, vv);
            stage_store4(kg, kv, vv);
        }
    }
    __syncthreads();

    const int t_tiles = tw32 / 16;
    for (int qt = qt_first; qt < q_tiles; qt += 4 * n_qg) {
        h8 qb[4];
        if (!FUSED && qt == qt_first) {
#pragma unroll
            for (int k4 = 0; k4 < 4; ++k4) qb[k4] = qb_first[k4];
        } else {
            load_q(qt, qb);
        }
        // S^T tiles: element r of st[j] is row t = 16j + 4g + r, column (query) c
        f4 st[TWM / 16];
        float mx = -INFINITY;
#pragma unroll
        for (int j = 0; j < TWM / 16; ++j) {
            st[j] = f4{0.f, 0.f, 0.f, 0.f};
            if (j < t_tiles) {
#pragma unroll
                for (int k4 = 0; k4 < 4; ++k4) {
                    h8 ka = *reinterpret_cast<const h8 *>(&ks[16 * j + c][32 * k4 + 8 * g]);
                    st[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qb[k4], st[j], 0, 0, 0);
                }
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int t = 16 * j + 4 * g + r;
                    const float sv = (t < cnt) ? st[j][r] * p.scale_log2 : -INFINITY;
                    st[j][r] = sv;
                    mx = fmaxf(mx, sv);
                }
            }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < TWM / 16; ++j) {
            if (j < t_tiles) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float e = exp2f(st[j][r] - mx);      // masked rows: exp2(-inf) = 0
                    st[j][r] = e;
                    sum += e;
                }
            }
        }
        sum += __shfl_xor(sum, 16, 64);
        sum += __shfl_xor(sum, 32, 64);

        // O^T tiles: element r of ot[dt] is row d = 16dt + 4g + r, column (query) c
        f4 ot[8];
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) ot[dt] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int jj = 0; jj < TWM / 32; ++jj) {
            if (2 * jj < t_tiles) {
                h8 pb;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    pb[r] = (half_t)st[2 * jj][r];
                    pb[4 + r] = (half_t)st[2 * jj + 1][r];
                }
#pragma unroll
                for (int dt = 0; dt < 8; ++dt) {
                    h8 va = *reinterpret_cast<const h8 *>(&vt[16 * dt + c][32 * jj + 8 * g]);
                    ot[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, pb, ot[dt], 0, 0, 0);
                }
            }
        }
        const int qrow = qt * 16 + c;
        if (qrow < p.Bq) {
            const long base = ((long)split * p.Hkv + hk) * p.Bq + qrow;
            float *po = p.part_o + base * ATT_D;
#pragma unroll
            for (int dt = 0; dt < 8; ++dt) {
                if (COHERENT) st_f4(po + 16 * dt + 4 * g, ot[dt]);
                else *reinterpret_cast<f4 *>(po + 16 * dt + 4 * g) = ot[dt];
            }
            if (g == 0) {
                if (COHERENT) { st_f32(p.part_ml + base * 2, mx); st_f32(p.part_ml + base * 2 + 1, sum); }
                else { p.part_ml[base * 2] = mx; p.part_ml[base * 2 + 1] = sum; }
            }
        }
    }
}

template <bool FUSED>
__global__ __launch_bounds__(256) void attn_prefix_kernel(AttnParams p) {
    attn_prefix_body<FUSED, false, ATT_TW_MAX>(p, blockIdx.x, blockIdx.y, blockIdx.z, gridDim.z);
}

// ---- causal attention of a prefill on the matrix cores ----------------------------------------------------------
// grid (ceil(S / 64), H): a workgroup owns 64 consecutive query positions of one head, wave w the 16 of them from
// 64 qb + 16 w.  It walks the key tiles (PF_TW rows, staged once per workgroup: K row-major, V transposed, as in
// attn_prefix_body) from position 0 to its diagonal with an online softmax: per tile S^T = K . Q^T and
// O^T += V^T . P^T on the matrix cores (the B operand of the second product is the accumulator layout of the first),
// running maximum / sum / O^T in registers, so nothing but the fp16 result is written.  The next tile's K / V rows
// are in flight (registers) while the current one is multiplied.  q [S,H,128], k, v [S,Hkv,128], out [S,H,128].
constexpr int PF_TW = 64;
struct PrefillParams {
    const half_t *q, *k, *v;
    half_t *out;
    int S, H, Hkv, n_rep;
    float scale_log2;
};

__global__ __launch_bounds__(256) void attn_prefill_kernel(PrefillParams p) {
    __shared__ __attribute__((aligned(16))) half_t ks[PF_TW][ATT_KPITCH];
    __shared__ __attribute__((aligned(16))) half_t vt[ATT_D][PF_TW + 8];
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63, c = lane & 15, g = lane >> 4;
    const int qb = gridDim.x - 1 - blockIdx.x, h = blockIdx.y, hk = h / p.n_rep;     // longest walks are dispatched first
    const int q_lo = 64 * qb + 16 * wave;                  // this wave's first query position
    const int my_q = q_lo + c;                             // this lane's query (column c of the tiles)
    const int last_key = min(64 * qb + 63, p.S - 1);       // the workgroup's diagonal
    const int n_tiles = last_key / PF_TW + 1;

    // B operand of S^T = K . Q^T: dims 32 k4 + 8g .. +7 of query row c
    h8 qbop[4];
    {
        const half_t *qp = p.q + ((long)min(my_q, p.S - 1) * p.H + h) * ATT_D + 8 * g;
#pragma unroll
        for (int k4 = 0; k4 < 4; ++k4) qbop[k4] = *reinterpret_cast<const h8 *>(qp + 32 * k4);
    }
    constexpr int PER = PF_TW * 16 / 256;                  // 16-byte pieces of K (and of V) per thread and tile
    u32x4 kreg[PER], vreg[PER];
    // a thread moves piece ch (8 dims) of FOUR consecutive keys, so that V goes to its transposed tile as 8-byte stores
    static_assert(PER == 4, "four keys per thread");
    auto tile_load = [&](int kt) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int t = 4 * (tid >> 4) + i, ch = tid & 15;
            const int row = kt * PF_TW + t;
            kreg[i] = u32x4{0, 0, 0, 0}; vreg[i] = u32x4{0, 0, 0, 0};
            if (row < p.S) {
                const long off = ((long)row * p.Hkv + hk) * ATT_D + ch * 8;
                kreg[i] = *reinterpret_cast<const u32x4 *>(p.k + off);
                vreg[i] = *reinterpret_cast<const u32x4 *>(p.v + off);
            }
        }
    };
    auto tile_store = [&]() {
        const int t0 = 4 * (tid >> 4), ch = tid & 15;
#pragma unroll
        for (int i = 0; i < PER; ++i) *reinterpret_cast<u32x4 *>(&ks[t0 + i][ch * 8]) = kreg[i];
        const int pos = vt_pos(t0);                            // keys t0 .. t0+3 sit side by side in a row of vt
        const h8 v0 = __builtin_bit_cast(h8, vreg[0]), v1 = __builtin_bit_cast(h8, vreg[1]);
        const h8 v2 = __builtin_bit_cast(h8, vreg[2]), v3 = __builtin_bit_cast(h8, vreg[3]);
#pragma unroll
        for (int j = 0; j < 8; ++j) *reinterpret_cast<h4 *>(&vt[ch * 8 + j][pos]) = h4{v0[j], v1[j], v2[j], v3[j]};
    };

    float m_run = -INFINITY, l_run = 0.f;                  // of query c (the same in the four lane groups)
    f4 ot[8];                                              // O^T: element r of ot[dt] is dim 16 dt + 4g + r of query c
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) ot[dt] = f4{0.f, 0.f, 0.f, 0.f};

    tile_load(0);
    for (int kt = 0; kt < n_tiles; ++kt) {
        __syncthreads();                                   // everyone is done with the previous tile
        tile_store();
        __syncthreads();
        if (kt + 1 < n_tiles) tile_load(kt + 1);
        const int k_lo = kt * PF_TW;
        if (k_lo > q_lo + 15) continue;                    // every key of this tile lies after this wave's queries
        // 16-row sub-tiles that hold a key <= the wave's last query
        const int subs = min(PF_TW / 16, (q_lo + 15 - k_lo) / 16 + 1);
        f4 st[PF_TW / 16];
        float mx = -INFINITY;
#pragma unroll
        for (int j = 0; j < PF_TW / 16; ++j) {
            st[j] = f4{0.f, 0.f, 0.f, 0.f};
            if (j < subs) {
#pragma unroll
                for (int k4 = 0; k4 < 4; ++k4) {
                    h8 ka = *reinterpret_cast<const h8 *>(&ks[16 * j + c][32 * k4 + 8 * g]);
                    st[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qbop[k4], st[j], 0, 0, 0);
                }
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int key = k_lo + 16 * j + 4 * g + r;
                const float sv = (j < subs && key <= my_q && key < p.S) ? st[j][r] * p.scale_log2 : -INFINITY;
                st[j][r] = sv;
                mx = fmaxf(mx, sv);
            }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx);              // finite from the first tile on: key 0 precedes every query
        const float alpha = exp2f(m_run - m_new);          // exp2(-inf) = 0 on the first tile
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < PF_TW / 16; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float e = exp2f(st[j][r] - m_new);
                st[j][r] = e;
                sum += e;
            }
        sum += __shfl_xor(sum, 16, 64);
        sum += __shfl_xor(sum, 32, 64);
        l_run = l_run * alpha + sum;
        m_run = m_new;
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) ot[dt] *= alpha;
#pragma unroll
        for (int jj = 0; jj < PF_TW / 32; ++jj) {
            if (2 * jj < subs) {
                h8 pb;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    pb[r] = (half_t)st[2 * jj][r];
                    pb[4 + r] = (half_t)st[2 * jj + 1][r];
                }
#pragma unroll
                for (int dt = 0; dt < 8; ++dt) {
                    h8 va = *reinterpret_cast<const h8 *>(&vt[16 * dt + c][32 * jj + 8 * g]);
                    ot[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, pb, ot[dt], 0, 0, 0);
                }
            }
        }
    }
    if (my_q < p.S) {
        const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
        half_t *op = p.out + ((long)my_q * p.H + h) * ATT_D;
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) {
            const h4 o = {(half_t)(ot[dt][0] * inv), (half_t)(ot[dt][1] * inv), (half_t)(ot[dt][2] * inv), (half_t)(ot[dt][3] * inv)};
            *reinterpret_cast<h4 *>(op + 16 * dt + 4 * g) = o;
        }
    }
}

// One wave per (branch b, query head h): the query heads of one kv head walk the same suffix rows in different
// waves (the rows come from the cache after the first), so a wave's chain of memory round trips does not grow with
// the number of query heads per kv head.  PARTIAL: the pass over the suffix and the new token leaves an un-normalised
// partial (split index p.splits) for the workgroup that merges, instead of folding in the prefix partials itself.
// sub, nsub: nsub consecutive waves of the workgroup share the query; wave `sub` of them walks every
// nsub-th group of four rows, so that a long suffix is a single batch of loads per wave instead of a chain of
// batches; the waves' results are folded through LDS (every wave of the workgroup must then make this call; a wave
// without a query of its own passes a valid (b, h) and live = false, and writes nothing).
template <bool FUSED, bool PARTIAL>
__device__ __forceinline__ void attn_suffix_body(const AttnParams &p, int b, int h, int sub = 0, int nsub = 1, bool live = true) {
    const int hk = div_rep(p, h);
    __shared__ __attribute__((aligned(16))) half_t s_kv[FUSED ? 4 : 1][3][ATT_D];     // FUSED: this wave's new k and v rows, its query
    __shared__ float s_fold[4][16][10];                                                 // nsub > 1: the waves' states (m, l, o[8])
    // Lane = 16 g + Q4_LPR rl + e.  In the Q4_0 walk below a row belongs to the Q4_LPR lanes (g, rl, 0..Q4_LPR-1), lane e
    // holding bytes (64 / Q4_LPR) e .. of it; everywhere else the 16 lanes of group g share a row in eight-dim pieces, lane
    // (rl, e) taking piece c = Q4_DW e + rl - a piece whose dims are among those the lane holds in the walk, so that the
    // walk's result needs no exchange between lanes with different e.
    // Measured (64 branches x 32 heads, ragged suffixes of 0..256 rows / 100 branches at ~55 rows): 8 lanes a row and 2 passes a
    // chunk 22.1 / 14.2 us; 4 lanes 23.6 / 16.2 (more registers, 64 lane exchanges at the end); 16 lanes 26.6 / 14.3; 4 passes
    // a chunk 23.9 / 15.8, 1 pass 23.7 / 13.8.  Before (16 lanes, 4 rows a batch, no request ahead): 28.6 / 14.8 us.
    constexpr int Q4_LPR = 8;                              // lanes per row (4, 8 or 16)
    constexpr int Q4_DW = 16 / Q4_LPR;                     // dwords of a row's 64 bytes per lane = row slots per group
    constexpr int Q4_ROWS = 4 * Q4_DW;                     // rows per pass of the wave
    constexpr int Q4_CH = 2;                               // passes per chunk
    const int lane = threadIdx.x & 63, g = lane >> 4, e = lane & (Q4_LPR - 1), rl = (lane & 15) / Q4_LPR, c = Q4_DW * e + rl;
    const int wave = threadIdx.x >> 6;
    int len = 0;
    // a length beyond the branch's rows (a device counter that ran past the cache) is cut at the cache's end
    if (p.suffix_format != SMH_KV_NONE) len = p.causal ? b + 1 : min(p.lens[(long)b * p.lens_stride], (int)p.suffix_batch_stride_rows);
    const int gg = g + 4 * sub, gstride = 4 * nsub;      // this group's first row and the distance to its next one
    const long row0 = (long)b * p.suffix_batch_stride_rows;     // first suffix row of this branch
    // pool row that holds suffix position t of this branch
    auto row_of = [&](int t) -> long {
        if (p.pages == nullptr) return row0 + t;
        const long i = (long)b * p.pages_stride + t;
        long id;
        if (p.page_bytes == 4) id = reinterpret_cast<const int32_t *>(p.pages)[i];
        else if (p.page_bytes == 2) id = reinterpret_cast<const int16_t *>(p.pages)[i];
        else id = reinterpret_cast<const int64_t *>(p.pages)[i];
        return min(max(id, 0L), p.pool_rows - 1);
    };
    // ---- Q4_0 suffix rows: a wave takes Q4_ROWS rows per pass (row slot Q4_DW g + rl) and Q4_CH passes per chunk; wave
    // `sub` of the nsub that share a query takes every nsub-th pass.  All loads of a chunk are requested together, and
    // the next chunk's before this one is used: the time of this walk is its dependent trips to memory (page id -> row)
    // and its instructions, not its bytes. ----
    typedef uint32_t q4_dw_t __attribute__((ext_vector_type(Q4_DW > 1 ? Q4_DW : 2)));
    struct Q4One { uint32_t x; __device__ uint32_t operator[](int) const { return x; } };
    typedef std::conditional_t<Q4_DW == 1, Q4One, q4_dw_t> q4_reg_t;
    struct Q4Chunk { q4_reg_t k[Q4_CH], v[Q4_CH]; uint32_t ks[Q4_CH], vs[Q4_CH]; };
    const int q4_passes = p.suffix_format == SMH_KV_Q40 ? (len + Q4_ROWS - 1) / Q4_ROWS : 0;     // passes over all waves of the query
    const int q4_mine = q4_passes > sub ? (q4_passes - sub + nsub - 1) / nsub : 0;                // passes of this wave
    const int q4_chunks = (q4_mine + Q4_CH - 1) / Q4_CH;
    auto q4_pos = [&](int n, int u) { return Q4_ROWS * (sub + nsub * (Q4_CH * n + u)) + Q4_DW * g + rl; };  // suffix position of this lane's row
    auto q4_ids = [&](int n, long (&id)[Q4_CH]) {
#pragma unroll
        for (int u = 0; u < Q4_CH; ++u) id[u] = row_of(min(q4_pos(n, u), len - 1));               // rows past the end repeat the last one
    };
    auto q4_rows = [&](const long (&id)[Q4_CH], Q4Chunk &ck) {
#pragma unroll
        for (int u = 0; u < Q4_CH; ++u) {
            const long row = id[u] * p.Hkv + hk;
            ck.k[u] = *reinterpret_cast<const q4_reg_t *>((const uint8_t *)p.suffix_k + row * 64 + 4 * Q4_DW * e);
            ck.v[u] = *reinterpret_cast<const q4_reg_t *>((const uint8_t *)p.suffix_v + row * 64 + 4 * Q4_DW * e);
            ck.ks[u] = *reinterpret_cast<const uint32_t *>(p.suffix_ks + row * 2);
            ck.vs[u] = *reinterpret_cast<const uint32_t *>(p.suffix_vs + row * 2);
        }
    };
    Q4Chunk q4_first;                                       // chunk 0, requested as early as the length is known
    long q4_next_id[Q4_CH];                                 // page ids of the chunk after the one in flight
    auto q4_prime = [&]() {
        if (q4_chunks > 0) {
            q4_ids(0, q4_next_id);
            q4_rows(q4_next_id, q4_first);
            if (q4_chunks > 1) q4_ids(1, q4_next_id);
        }
    };
    RowRegs q_first;
    int pos = 0;
    if (FUSED) {
        // Two round trips to memory, not more: first everything that depends on no other load - the suffix length
        // (requested above), the position, the suffix index and the slabs of q, k and v (lane owns the rotation pair
        // (lane, lane + 64) of each: 2 x ksplit loads of 4 bytes; read in the row layout, 8 dims a lane, q's slabs
        // alone take 128 registers and the requests leave one after the other) - then what depends on the length
        // (the first batch of rows) and on the position (the rotation factors).  q changes to the row layout
        // through LDS; k is rotated, k and v are appended to the branch's suffix cache as Q4_0 and left in LDS as
        // exact fp16 for the pass below.
        pos = *p.pos_dev;
        int t = -1;
        SlabColumn cq1, cq2, ck1, ck2, cv1, cv2;
        qkv_request(p, b, h * ATT_D + lane, cq1);
        qkv_request(p, b, h * ATT_D + lane + 64, cq2);
        if (sub == 0) {                                            // the wave that owns the new token
            t = p.app_k != nullptr ? *p.app_t : -1;
            const int kcol = (p.H + hk) * ATT_D, vcol = (p.H + p.Hkv + hk) * ATT_D;
            qkv_request(p, b, kcol + lane, ck1); qkv_request(p, b, kcol + lane + 64, ck2);
            qkv_request(p, b, vcol + lane, cv1); qkv_request(p, b, vcol + lane + 64, cv2);
        }
        q4_prime();
        const half_t cos_l = p.cos_tab[(long)pos * 64 + lane], sin_l = p.sin_tab[(long)pos * 64 + lane];
        half_t q1 = qkv_sum(cq1), q2 = qkv_sum(cq2);
        half_t k1 = q1, k2 = q1, v1 = q1, v2 = q1;
        if (sub == 0) { k1 = qkv_sum(ck1); k2 = qkv_sum(ck2); v1 = qkv_sum(cv1); v2 = qkv_sum(cv2); }
        rope_pair2(q1, q2, cos_l, sin_l);
        s_kv[wave][2][lane] = q1; s_kv[wave][2][lane + 64] = q2;
        asm volatile("" ::: "memory");                              // the reads below are of another type: keep them behind the writes
        q_first = row_from_fp16(&s_kv[wave][2][0], c);             // same wave writes and reads: LDS operations complete in order
        if (sub == 0) {
            rope_pair2(k1, k2, cos_l, sin_l);
            if (live && h == hk * p.n_rep && t >= 0 && t < p.app_smax) {     // the first query head of a kv head appends the rows
                const long row = ((long)b * p.app_smax + t) * p.Hkv + hk;
                kv_store_row2(k1, k2, p.app_k + row * 64, p.app_ks + row * 2, lane);
                kv_store_row2(v1, v2, p.app_v + row * 64, p.app_vs + row * 2, lane);
            }
            s_kv[wave][0][lane] = k1; s_kv[wave][0][lane + 64] = k2;
            s_kv[wave][1][lane] = v1; s_kv[wave][1][lane + 64] = v2;
            asm volatile("" ::: "memory");
            // same wave writes and reads: LDS operations of a wave complete in order
        }
    }

    {
        RowRegs qr;
        if (!FUSED) qr = row_from_fp16(p.q + ((long)b * p.H + h) * ATT_D, c);
        else qr = q_first;
        SoftState st;
        st.m = -INFINITY;
        st.l = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) st.o[j] = 0.f;

        // Every load below is issued before its first use, a batch at a time: a wave has few rows to visit
        // (tens, a quarter each per group), so its time is the number of memory round trips it makes in a row.
        // ---- loads for the end of the pass: the new token's exact K/V, the first two prefix partials ----
        const int qrow = b * p.n_rep + (h - hk * p.n_rep);
        const bool has_cur = (FUSED || p.cur_k != nullptr) && g == 0 && sub == 0;
        RowRegs cur_kr = qr, cur_vr = qr;
        if (has_cur) {
            if (FUSED) {
                cur_kr = row_from_fp16(&s_kv[wave][0][0], c);
                cur_vr = row_from_fp16(&s_kv[wave][1][0], c);
            } else {
                const long off = ((long)b * p.Hkv + hk) * ATT_D;
                cur_kr = row_from_fp16(p.cur_k + off, c);
                cur_vr = row_from_fp16(p.cur_v + off, c);
            }
        }
        constexpr int PRE = 2;
        f4 pre_lo[PRE], pre_hi[PRE];
        float pre_m[PRE], pre_l[PRE];
#pragma unroll
        for (int i = 0; i < PRE; ++i) {
            const int sp = gg + gstride * i;
            if (!PARTIAL && sp < p.splits) {
                const long base = ((long)sp * p.Hkv + hk) * p.Bq + qrow;
                pre_lo[i] = *reinterpret_cast<const f4 *>(p.part_o + base * ATT_D + 4 * c);
                pre_hi[i] = *reinterpret_cast<const f4 *>(p.part_o + base * ATT_D + 64 + 4 * c);
                pre_m[i] = p.part_ml[base * 2];
                pre_l[i] = p.part_ml[base * 2 + 1];
            }
        }
        // ---- this branch's suffix: group g takes rows g, g+4, ... in batches ----
        if (p.suffix_format == SMH_KV_FP16) {
            constexpr int U = 4;
            for (int t0 = gg; t0 < len; t0 += gstride * U) {
                RowRegs kr[U], vr[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const long off = row_of(min(t0 + gstride * u, len - 1)) * p.sfx_row_stride + (long)hk * p.sfx_head_stride;
                    kr[u] = row_from_fp16((const half_t *)p.suffix_k + off, c);
                    vr[u] = row_from_fp16((const half_t *)p.suffix_v + off, c);
                }
#pragma unroll
                for (int u = 0; u < U; ++u)
                    if (t0 + gstride * u < len) soft_add_row(st, row_dot(kr[u], qr) * p.scale_log2, vr[u]);
            }
        } else if (q4_chunks > 0) {
            if (!FUSED) q4_prime();
            RowRegs qj[Q4_DW];                              // the query's dims this lane holds of a row: pieces Q4_DW e + j
#pragma unroll
            for (int j = 0; j < Q4_DW; ++j)
                qj[j] = FUSED ? row_from_fp16(&s_kv[wave][2][0], Q4_DW * e + j) : row_from_fp16(p.q + ((long)b * p.H + h) * ATT_D, Q4_DW * e + j);
            float m = -INFINITY, l = 0.f;                   // m: common to the group; l, o: of this lane's row slot
            float o[Q4_DW][8];
#pragma unroll
            for (int j = 0; j < Q4_DW; ++j)
#pragma unroll
                for (int k = 0; k < 8; ++k) o[j][k] = 0.f;
            Q4Chunk cur = q4_first;
            for (int n = 0; n < q4_chunks; ++n) {
                Q4Chunk nxt;
                if (n + 1 < q4_chunks) {
                    q4_rows(q4_next_id, nxt);
                    if (n + 2 < q4_chunks) q4_ids(n + 2, q4_next_id);
                }
                float sc[Q4_CH];
#pragma unroll
                for (int u = 0; u < Q4_CH; ++u) {
                    float d = 0.f;
#pragma unroll
                    for (int j = 0; j < Q4_DW; ++j) {
                        const RowRegs kr = row_from_q40(cur.k[u][j], cur.ks[u]);
                        d = __builtin_amdgcn_fdot2(kr.a02, qj[j].a02, d, false);
                        d = __builtin_amdgcn_fdot2(kr.a13, qj[j].a13, d, false);
                        d = __builtin_amdgcn_fdot2(kr.b02, qj[j].b02, d, false);
                        d = __builtin_amdgcn_fdot2(kr.b13, qj[j].b13, d, false);
                    }
                    d += dpp_move<DPP_QUAD_XOR1>(d);        // the lanes that share the row
                    d += dpp_move<DPP_QUAD_XOR2>(d);
                    if (Q4_LPR >= 8) d += dpp_move<DPP_ROW_HALF_MIRROR>(d);
                    if (Q4_LPR == 16) d += dpp_move<DPP_ROW_ROR8>(d);
                    sc[u] = q4_pos(n, u) < len ? d * p.scale_log2 : -INFINITY;
                }
                float mx = sc[0];
#pragma unroll
                for (int u = 1; u < Q4_CH; ++u) mx = fmaxf(mx, sc[u]);
                if (Q4_LPR <= 8) mx = fmaxf(mx, dpp_move<DPP_ROW_ROR8>(mx)); // the row slots of the group
                if (Q4_LPR == 4) mx = fmaxf(mx, dpp_move<DPP_ROW_ROR4>(mx));
                const float m_new = fmaxf(m, mx);
                const float m_ref = m_new == -INFINITY ? 0.f : m_new;    // a group without a row yet: every factor below is exp2(-inf) = 0
                const float corr = exp2f(m - m_ref);
                m = m_new;
                l *= corr;
#pragma unroll
                for (int j = 0; j < Q4_DW; ++j)
#pragma unroll
                    for (int k = 0; k < 8; ++k) o[j][k] *= corr;
#pragma unroll
                for (int u = 0; u < Q4_CH; ++u) {
                    const float pr = exp2f(sc[u] - m_ref);
                    l += pr;
#pragma unroll
                    for (int j = 0; j < Q4_DW; ++j) {
                        const RowRegs vr = row_from_q40(cur.v[u][j], cur.vs[u]);
                        o[j][0] += pr * (float)vr.a02.x; o[j][1] += pr * (float)vr.a02.y;
                        o[j][2] += pr * (float)vr.a13.x; o[j][3] += pr * (float)vr.a13.y;
                        o[j][4] += pr * (float)vr.b02.x; o[j][5] += pr * (float)vr.b02.y;
                        o[j][6] += pr * (float)vr.b13.x; o[j][7] += pr * (float)vr.b13.y;
                    }
                }
                cur = nxt;
            }
            // the group's row slots added up, then lane (rl, e) keeps piece Q4_DW e + rl = c
            if (Q4_LPR <= 8) l += dpp_move<DPP_ROW_ROR8>(l);
            if (Q4_LPR == 4) l += dpp_move<DPP_ROW_ROR4>(l);
#pragma unroll
            for (int j = 0; j < Q4_DW; ++j)
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    if (Q4_LPR <= 8) o[j][k] += dpp_move<DPP_ROW_ROR8>(o[j][k]);
                    if (Q4_LPR == 4) o[j][k] += dpp_move<DPP_ROW_ROR4>(o[j][k]);
                }
            st.m = m;
            st.l = l;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                float v = o[0][k];
#pragma unroll
                for (int j = 1; j < Q4_DW; ++j) v = rl == j ? o[j][k] : v;
                st.o[k] = v;
            }
        }
        // ---- the new token's exact K/V (group 0 only) ----
        if (has_cur) soft_add_row(st, row_dot(cur_kr, qr) * p.scale_log2, cur_vr);
        // ---- prefix partials: the group folds in splits gg, gg + gstride, ... ----
#pragma unroll
        for (int i = 0; i < PRE; ++i) {
            if (!PARTIAL && gg + gstride * i < p.splits) {
                const float o2[8] = {pre_lo[i][0], pre_lo[i][2], pre_lo[i][1], pre_lo[i][3], pre_hi[i][0], pre_hi[i][2], pre_hi[i][1], pre_hi[i][3]};
                soft_merge(st, pre_m[i], pre_l[i], o2);
            }
        }
        for (int sp = gg + gstride * PRE; !PARTIAL && sp < p.splits; sp += gstride) {
            const long base = ((long)sp * p.Hkv + hk) * p.Bq + qrow;
            const f4 lo = *reinterpret_cast<const f4 *>(p.part_o + base * ATT_D + 4 * c);
            const f4 hi = *reinterpret_cast<const f4 *>(p.part_o + base * ATT_D + 64 + 4 * c);
            const float o2[8] = {lo[0], lo[2], lo[1], lo[3], hi[0], hi[2], hi[1], hi[3]};
            soft_merge(st, p.part_ml[base * 2], p.part_ml[base * 2 + 1], o2);
        }
        // ---- merge the four groups (xor 16, xor 32) ----
#pragma unroll
        for (int sh = 16; sh <= 32; sh <<= 1) {
            const float m2 = __shfl_xor(st.m, sh, 64);
            const float l2 = __shfl_xor(st.l, sh, 64);
            float o2[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) o2[j] = __shfl_xor(st.o[j], sh, 64);
            soft_merge(st, m2, l2, o2);
        }
        if (nsub > 1) {                                // (uniform over the workgroup)
            if (g == 0) {
                float *mine = s_fold[wave][c];
                mine[0] = st.m; mine[1] = st.l;
#pragma unroll
                for (int j = 0; j < 8; ++j) mine[2 + j] = st.o[j];
            }
            __syncthreads();
            if (g == 0 && sub == 0)
                for (int k = 1; k < nsub; ++k) soft_merge(st, s_fold[wave + k][c][0], s_fold[wave + k][c][1], &s_fold[wave + k][c][2]);
        }
        if (g == 0 && PARTIAL) {
            if (sub != 0 || !live) return;
            const long base = ((long)p.splits * p.Hkv + hk) * p.Bq + qrow;
            st_f4(p.part_o + base * ATT_D + 4 * c, f4{st.o[0], st.o[2], st.o[1], st.o[3]});
            st_f4(p.part_o + base * ATT_D + 64 + 4 * c, f4{st.o[4], st.o[6], st.o[5], st.o[7]});
            if (c == 0) { st_f32(p.part_ml + base * 2, st.m); st_f32(p.part_ml + base * 2 + 1, st.l); }
        } else if (g == 0 && sub == 0 && live) {
            const float inv = st.l > 0.f ? 1.0f / st.l : 0.f;
            half_t *op = p.out + ((long)b * p.H + h) * ATT_D;
            h4 lo = {(half_t)(st.o[0] * inv), (half_t)(st.o[2] * inv), (half_t)(st.o[1] * inv), (half_t)(st.o[3] * inv)};
            h4 hi = {(half_t)(st.o[4] * inv), (half_t)(st.o[6] * inv), (half_t)(st.o[5] * inv), (half_t)(st.o[7] * inv)};
            *reinterpret_cast<h4 *>(op + 4 * c) = lo;
            *reinterpret_cast<h4 *>(op + 64 + 4 * c) = hi;
        }
    }
}

template <bool FUSED>
__global__ __launch_bounds__(256) void attn_suffix_kernel(AttnParams p) {
    // suffix_waves (1, 2 or 4) waves per (branch, query head): more than one while branches x heads leave CUs idle.
    // Workgroups are dealt round-robin to the 8 XCDs (8 L2s); the heads of one branch share the 128-byte lines of that
    // branch's scales (2 fp16 per head and position), so ALL workgroups of a branch go to one XCD: workgroup L of the 1-D
    // grid sits on XCD L % 8 and takes branch 8 (L / 8 / per_branch) + L % 8, head group (L / 8) % per_branch.
    const int wave = threadIdx.x >> 6, nsub = p.suffix_waves;
    const int per_branch = (p.H * nsub + 3) >> 2;              // workgroups (four waves) per branch
    const int L = blockIdx.x, j = L >> 3;
    const int grp = j / per_branch;
    const int b = 8 * grp + (L & 7);
    if (b >= p.B) return;
    const int hq = (j - grp * per_branch) * 4 + wave;
    const int h = nsub == 4 ? hq >> 2 : (nsub == 2 ? hq >> 1 : hq);
    if (nsub == 1 && h >= p.H) return;
    // with shared queries every wave reaches the fold's barrier: one past the last head repeats it and writes nothing
    attn_suffix_body<FUSED, false>(p, b, min(h, p.H - 1), hq & (nsub - 1), nsub, h < p.H);
}

// ---- the whole decode attention in ONE launch -----------------------------------------------------------------
// grid (splits + ceil(Bq / per_wg), kv heads): workgroups x < splits take a slice of the prefix, the others the suffix
// + new token of per_wg = 1, 2 or 4 of the kv head's Bq = B x n_rep queries (4, 2 or 1 waves per query: with few
// queries a query's rows are spread over the waves, which shortens the longest chain of loads in the launch).  Every workgroup leaves partials with device-scope
// stores and counts itself in on the counters of the query tiles (16 queries of a kv head) it contributed to;
// the workgroup that completes a tile's count merges that tile's partials in split order (so the result does
// not depend on which workgroup that is), normalises and writes the output.  Nobody waits for anybody.
// FUSED: q and the new token's k, v come from the wq|wk|wv slabs (up to 16 branches); otherwise from p.q, p.cur_k/v.
constexpr int ATT_ONE_MAX_TILES = ATT_FUSED_MAX_Q / 16;

template <bool FUSED>
__global__ __launch_bounds__(256, 2) void attn_one_kernel(AttnParams p) {
    __shared__ uint32_t s_last[ATT_ONE_MAX_TILES];
    const int hk = blockIdx.y;
    const int tid = threadIdx.x;
    const int q_tiles = (p.Bq + 15) / 16;
    const int sw_shift = p.suffix_waves == 4 ? 2 : (p.suffix_waves == 2 ? 1 : 0);
    const int per_wg = 4 >> sw_shift;          // queries of one suffix workgroup (suffix_waves = 1, 2 or 4 waves each)
    int tile_lo = 0, tile_hi = q_tiles - 1;    // query tiles this workgroup contributed to
    if ((int)blockIdx.x < p.splits) {
        attn_prefix_body<FUSED, true, ATT_ONE_TW>(p, blockIdx.x, hk);
    } else {
        const int j = (int)blockIdx.x - p.splits, wave_ = tid >> 6;
        const int qrow = per_wg * j + (wave_ >> sw_shift);        // query of this kv head: branch qrow / n_rep, its query head qrow % n_rep
        const int qc = min(qrow, p.Bq - 1);
        attn_suffix_body<FUSED, true>(p, div_rep(p, qc), hk * p.n_rep + mod_rep(p, qc), wave_ & (p.suffix_waves - 1), p.suffix_waves, qrow < p.Bq);
        tile_lo = tile_hi = (per_wg * j) / 16;  // a workgroup's 1, 2 or 4 consecutive queries never straddle a tile of 16
    }
    wait_vmem();                               // this wave's partials have reached memory ...
    __syncthreads();                           // ... and those of the whole workgroup
    if (tid < q_tiles) {
        uint32_t last = 0u;
        if (tid >= tile_lo && tid <= tile_hi) {
            // arrivals a tile waits for: every prefix slice + the suffix workgroups whose queries fall into it
            const int pw_shift = 2 - sw_shift;       // per_wg = 1 << pw_shift
            const int j_lo = (16 * tid) >> pw_shift, j_hi = (min(p.Bq, 16 * tid + 16) - 1) >> pw_shift;
            const uint32_t expected = (uint32_t)(p.splits + j_hi - j_lo + 1);
            uint32_t *cnt = p.counters + hk * q_tiles + tid;
            const uint32_t prev = __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (prev == expected - 1u) {
                st_u32(cnt, 0u);               // ready for the next launch
                last = 1u;
            }
        }
        s_last[tid] = last;
    }
    __syncthreads();

    // ---- merge the completed tiles: 16 lanes per query (dims 4cc.. and 64+4cc..), 16 groups of 16 lanes ----
    // A tile of nq queries (npow = nq rounded up to a power of two) gives each query sub = 16 / npow consecutive
    // groups; group `si` of a query folds partials si, si + sub, ... (its loads go out together, four partials at
    // a time).  The groups of a query are then folded within their wave by lane exchange and across waves through
    // LDS.  The order depends only on the shape, not on which workgroup merges.
    __shared__ float s_merge[4][16][10];
    const int cc = tid & 15, gi = tid >> 4, wave = tid >> 6;
    const int n_part = p.splits + 1;
    for (int qt = tile_lo; qt <= tile_hi; ++qt) {
        if (s_last[qt] == 0u) continue;                       // (uniform over the workgroup)
        const int nq = min(16, p.Bq - 16 * qt);
        int npow = 1;
        while (npow < nq) npow <<= 1;
        const int sub = 16 / npow;
        const int qi = gi / sub, si = gi & (sub - 1);
        const int qrow = 16 * qt + qi;
        const bool live = qi < nq;
        float m = -INFINITY, l = 0.f;
        float o[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = 0.f;
        auto fold = [&](float pm, float pl, const float (&po)[8]) {
            const float m_new = fmaxf(m, pm);
            if (m_new != -INFINITY) {
                const float c1 = exp2f(m - m_new), c2 = exp2f(pm - m_new);
                m = m_new;
                l = l * c1 + pl * c2;
#pragma unroll
                for (int j = 0; j < 8; ++j) o[j] = o[j] * c1 + po[j] * c2;
            }
        };
        for (int s0 = si; live && s0 < n_part; s0 += 4 * sub) {
            f4 lo[4], hi[4];
            float pm[4], pl[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (s0 + u * sub < n_part) {
                    const long base = ((long)(s0 + u * sub) * p.Hkv + hk) * p.Bq + qrow;
                    lo[u] = ld_f4(p.part_o + base * ATT_D + 4 * cc);
                    hi[u] = ld_f4(p.part_o + base * ATT_D + 64 + 4 * cc);
                    pm[u] = ld_f32(p.part_ml + base * 2);
                    pl[u] = ld_f32(p.part_ml + base * 2 + 1);
                }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if (s0 + u * sub < n_part) {
                    const float po[8] = {lo[u][0], lo[u][1], lo[u][2], lo[u][3], hi[u][0], hi[u][1], hi[u][2], hi[u][3]};
                    fold(pm[u], pl[u], po);
                }
            }
        }
        // groups of one wave (sub >= 2: neighbours, sub >= 4: all four); every lane of the wave takes part
        for (int sh = 16; sh <= 32 && sh < 16 * sub; sh <<= 1) {
            const float m2 = __shfl_xor(m, sh, 64), l2 = __shfl_xor(l, sh, 64);
            float o2[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) o2[j] = __shfl_xor(o[j], sh, 64);
            fold(m2, l2, o2);
        }
        if (sub > 4) {                                        // a query spans sub / 4 waves (uniform over the workgroup)
            if ((gi & 3) == 0) {
                float *mine = s_merge[wave][cc];
                mine[0] = m; mine[1] = l;
#pragma unroll
                for (int j = 0; j < 8; ++j) mine[2 + j] = o[j];
            }
            __syncthreads();
            if (si == 0 && live) {
                for (int k = 1; k < sub / 4; ++k) {
                    const float *other = s_merge[wave + k][cc];
                    const float po[8] = {other[2], other[3], other[4], other[5], other[6], other[7], other[8], other[9]};
                    fold(other[0], other[1], po);
                }
            }
            __syncthreads();                                  // s_merge is free for the next tile
        }
        if (si != 0 || !live) continue;
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        const int b = div_rep(p, qrow), h = hk * p.n_rep + mod_rep(p, qrow);
        half_t *op = p.out + ((long)b * p.H + h) * ATT_D;
        *reinterpret_cast<h4 *>(op + 4 * cc) = h4{(half_t)(o[0] * inv), (half_t)(o[1] * inv), (half_t)(o[2] * inv), (half_t)(o[3] * inv)};
        *reinterpret_cast<h4 *>(op + 64 + 4 * cc) = h4{(half_t)(o[4] * inv), (half_t)(o[5] * inv), (half_t)(o[6] * inv), (half_t)(o[7] * inv)};
    }
}

static int attn_plan_tw(int P, int Hkv) {
    // rows of the prefix per workgroup: as large as fits while still giving the 256 CUs work
    int tw = ATT_TW_MAX;
    while (tw > 32 && (long)((P + tw - 1) / tw) * Hkv < 256) tw >>= 1;
    return tw;
}

// Two launches: rows of the prefix per workgroup and the number of workgroups that share one slice's query tiles.
// Every slice leaves a partial per query, so wide slices mean less partial traffic; the CUs are filled first by
// dealing the rounds of query tiles (four tiles, one per wave) of a slice to several workgroups, which re-read the
// slice from the cache but write nothing extra, and only then by narrower slices.
static void attn_plan(int P, int Hkv, int Bq, int *tw_out, int *qgroups_out) {
    const int rounds = ((Bq + 15) / 16 + 3) / 4;
    constexpr int wgs_least = 256;
    int tw = ATT_TW_MAX, qg = 1;
    while ((long)((P + tw - 1) / tw) * Hkv * qg < wgs_least) {
        if (qg < rounds) qg = min(rounds, 2 * qg);
        else if (tw > 32) tw >>= 1;
        else break;
    }
    *tw_out = tw;
    *qgroups_out = qg;
}

// Suffix launch of the two-launch form: waves per (branch, query head) - more than one while the launch still fits
// the GPU in one round (4 waves of this kernel per SIMD, 1024 SIMDs).
static int attn_plan_suffix_waves_two(long queries) {
    int nsub = 4;
    constexpr int cap = 4096;                  // measured again with the 8-lanes-a-row walk: 2048 and 8192 are both slower
    while (nsub > 1 && queries * nsub > cap) nsub >>= 1;
    return nsub;
}

// One-launch kernel: waves that share a query's suffix rows - as many as keep the launch within one round of
// workgroups (two fit a compute unit).
static int attn_plan_suffix_waves(int splits, int Bq, int Hkv) {
    int nsub = 4;
    while (nsub > 1 && (long)(splits + (Bq + 4 / nsub - 1) / (4 / nsub)) * Hkv > 512) nsub >>= 1;
    return nsub;
}

}  // namespace smh

extern "C" size_t smh_attn_workspace_bytes(int B, int H, int P) {
    if (P <= 0 || B <= 0 || H <= 0) return 256;
    size_t splits = (size_t)(P + 31) / 32;          // worst case: 32 rows per workgroup
    return splits * (size_t)B * (size_t)H * (smh::ATT_D + 2) * sizeof(float) + 256;
}

constexpr size_t ATT_COUNTER_BYTES = 4096;     // one-launch variants: arrival counters at the start of the workspace

// what the paged entry point adds to the arguments of smh_shared_prefix_attn (zero strides: token-major tensors)
struct AttnExtras {
    const void *pages = nullptr;
    long pages_stride = 0;
    int page_bytes = 4;
    long pool_rows = 0;
    long pfx_row = 0, pfx_head = 0, sfx_row = 0, sfx_head = 0;
};

static int shared_prefix_attn(const char *who, bool one, const void *q, void *out, int B, int H, int Hkv, int D,
                              const void *prefix_k, const void *prefix_v, int P,
                              int suffix_format, const void *suffix_k, const void *suffix_v,
                              const void *suffix_ks, const void *suffix_vs, int Smax,
                              const int32_t *lens, int lens_stride, const void *cur_k, const void *cur_v,
                              void *workspace, size_t workspace_bytes, smh_stream_t stream, const AttnExtras &ex = AttnExtras()) {
    using namespace smh;
    SMH_REQUIRE(D == ATT_D, "%s: head dim %d (only 128)", who, D);
    SMH_REQUIRE(B >= 0 && B <= 65535 && H > 0 && Hkv > 0 && H % Hkv == 0 && P >= 0, "%s: B=%d (at most 65535) H=%d Hkv=%d P=%d", who, B, H, Hkv, P);
    SMH_REQUIRE(suffix_format == SMH_KV_NONE || suffix_format == SMH_KV_FP16 || suffix_format == SMH_KV_Q40,
                "%s: suffix_format=%d", who, suffix_format);
    if (B == 0) return 0;
    SMH_REQUIRE(q && out, "%s: null q/out", who);
    SMH_REQUIRE(P == 0 || (prefix_k && prefix_v), "%s: null prefix", who);
    if (suffix_format != SMH_KV_NONE) {
        SMH_REQUIRE(suffix_k && suffix_v && lens && Smax > 0 && (lens_stride == 0 || lens_stride == 1),
                    "%s: suffix arguments incomplete", who);
        SMH_REQUIRE(suffix_format != SMH_KV_Q40 || (suffix_ks && suffix_vs), "%s: null suffix scales", who);
    }
    SMH_REQUIRE((cur_k == nullptr) == (cur_v == nullptr), "%s: cur_k/cur_v must both be given or both be null", who);
    AttnParams p{};
    p.q = (const half_t *)q; p.out = (half_t *)out;
    p.prefix_k = (const half_t *)prefix_k; p.prefix_v = (const half_t *)prefix_v;
    p.suffix_k = suffix_k; p.suffix_v = suffix_v;
    p.suffix_ks = (const half_t *)suffix_ks; p.suffix_vs = (const half_t *)suffix_vs;
    p.lens = lens; p.lens_stride = lens_stride;
    p.cur_k = (const half_t *)cur_k; p.cur_v = (const half_t *)cur_v;
    p.suffix_batch_stride_rows = Smax;
    p.pages = ex.pages; p.pages_stride = ex.pages_stride; p.page_bytes = ex.page_bytes; p.pool_rows = ex.pool_rows;
    p.pfx_row_stride = ex.pfx_row ? ex.pfx_row : (long)Hkv * ATT_D; p.pfx_head_stride = ex.pfx_head ? ex.pfx_head : ATT_D;
    p.sfx_row_stride = ex.sfx_row ? ex.sfx_row : (long)Hkv * ATT_D; p.sfx_head_stride = ex.sfx_head ? ex.sfx_head : ATT_D;
    p.B = B; p.H = H; p.Hkv = Hkv; p.n_rep = H / Hkv; p.Bq = B * p.n_rep;
    p.P = P; p.suffix_format = suffix_format; p.causal = 0;
    p.scale_log2 = LOG2E / sqrtf((float)D);
    int qgroups = 1;
    if (one) p.tw = min(attn_plan_tw(P, Hkv), ATT_ONE_TW);
    else attn_plan(P, Hkv, p.Bq, &p.tw, &qgroups);
    p.splits = P > 0 ? (P + p.tw - 1) / p.tw : 0;
    if (one) {
        p.suffix_waves = attn_plan_suffix_waves(p.splits, p.Bq, Hkv);
        const int q_tiles = (p.Bq + 15) / 16;
        SMH_REQUIRE(q_tiles <= ATT_ONE_MAX_TILES && (size_t)Hkv * q_tiles * sizeof(uint32_t) <= ATT_COUNTER_BYTES,
                    "%s: %d queries per kv head (at most %d), %d kv heads", who, p.Bq, ATT_FUSED_MAX_Q, Hkv);
        size_t n_part = (size_t)(p.splits + 1) * Hkv * p.Bq;
        size_t need = ATT_COUNTER_BYTES + n_part * (ATT_D + 2) * sizeof(float);
        SMH_REQUIRE(workspace && workspace_bytes >= need, "%s: workspace %zu < %zu bytes", who, workspace_bytes, need);
        p.counters = (uint32_t *)workspace;
        p.part_o = (float *)((char *)workspace + ATT_COUNTER_BYTES);
        p.part_ml = p.part_o + n_part * ATT_D;
        hipLaunchKernelGGL(attn_one_kernel<false>, dim3(p.splits + (p.Bq + 4 / p.suffix_waves - 1) / (4 / p.suffix_waves), Hkv), dim3(256), 0, (hipStream_t)stream, p);
        return launch_status();
    }
    size_t n_part = (size_t)p.splits * Hkv * p.Bq;
    SMH_REQUIRE(p.splits == 0 || (workspace && workspace_bytes >= n_part * (ATT_D + 2) * sizeof(float)),
                "%s: workspace %zu < %zu bytes", who, workspace_bytes, n_part * (ATT_D + 2) * sizeof(float));
    p.part_o = (float *)workspace;
    p.part_ml = p.part_o + n_part * ATT_D;
    if (p.splits > 0)
        hipLaunchKernelGGL(attn_prefix_kernel<false>, dim3(p.splits, Hkv, qgroups), dim3(256), 0, (hipStream_t)stream, p);
    p.suffix_waves = attn_plan_suffix_waves_two((long)B * H);
    hipLaunchKernelGGL(attn_suffix_kernel<false>, dim3((unsigned)(((H * p.suffix_waves + 3) / 4) * ((B + 7) / 8 * 8))), dim3(256), 0, (hipStream_t)stream, p);
    return launch_status();
}

extern "C" int smh_shared_prefix_attn(const void *q, void *out, int B, int H, int Hkv, int D,
                                      const void *prefix_k, const void *prefix_v, int P,
                                      int suffix_format, const void *suffix_k, const void *suffix_v,
                                      const void *suffix_ks, const void *suffix_vs, int Smax,
                                      const int32_t *lens, int lens_stride, const void *cur_k, const void *cur_v,
                                      void *workspace, size_t workspace_bytes, smh_stream_t stream) {
    return shared_prefix_attn("smh_shared_prefix_attn", false, q, out, B, H, Hkv, D, prefix_k, prefix_v, P, suffix_format, suffix_k,
                              suffix_v, suffix_ks, suffix_vs, Smax, lens, lens_stride, cur_k, cur_v, workspace, workspace_bytes, stream);
}

extern "C" int smh_paged_prefix_attn(const void *q, void *out, int B, int H, int Hkv, int D,
                                     const void *prefix_k, const void *prefix_v, int P, long prefix_row_stride, long prefix_head_stride,
                                     int pool_format, const void *pool_k, const void *pool_v, const void *pool_ks, const void *pool_vs,
                                     long pool_row_stride, long pool_head_stride, long pool_rows,
                                     const void *pages, int page_bytes, long pages_stride, int pages_cols, const int32_t *lens, int lens_stride,
                                     const void *cur_k, const void *cur_v, int single_launch,
                                     void *workspace, size_t workspace_bytes, smh_stream_t stream) {
    using namespace smh;
    const char *who = "smh_paged_prefix_attn";
    SMH_REQUIRE(pages_cols >= 1 && pages_cols <= pages_stride, "%s: pages_cols=%d must lie in 1 .. pages_stride=%ld", who, pages_cols, pages_stride);
    SMH_REQUIRE(pool_format == SMH_KV_FP16 || pool_format == SMH_KV_Q40, "%s: pool_format=%d", who, pool_format);
    SMH_REQUIRE(pages != nullptr && (page_bytes == 2 || page_bytes == 4 || page_bytes == 8) && pages_stride >= 1,
                "%s: pages=%p page_bytes=%d (2, 4 or 8) pages_stride=%ld", who, pages, page_bytes, pages_stride);
    SMH_REQUIRE(pages_stride <= 0x7fffffffL, "%s: pages_stride=%ld", who, pages_stride);
    SMH_REQUIRE(pool_rows >= 1, "%s: pool_rows=%ld", who, pool_rows);
    SMH_REQUIRE(prefix_row_stride >= 0 && prefix_head_stride >= 0 && pool_row_stride >= 0 && pool_head_stride >= 0 &&
                prefix_row_stride % 8 == 0 && prefix_head_stride % 8 == 0 && pool_row_stride % 4 == 0 && pool_head_stride % 4 == 0,
                "%s: strides must be non-negative (0 = token-major), prefix strides multiples of 8 and pool strides multiples of 4 elements", who);
    SMH_REQUIRE(pool_format != SMH_KV_Q40 || (pool_row_stride == 0 && pool_head_stride == 0), "%s: Q4_0 pools are token-major (strides 0)", who);
    AttnExtras ex;
    ex.pages = pages; ex.page_bytes = page_bytes; ex.pages_stride = pages_stride; ex.pool_rows = pool_rows;
    ex.pfx_row = prefix_row_stride; ex.pfx_head = prefix_head_stride; ex.sfx_row = pool_row_stride; ex.sfx_head = pool_head_stride;
    // (the kernels cut lens[b] to the row count they are given: the ids a table row holds, not the distance between rows)
    return shared_prefix_attn(who, single_launch != 0, q, out, B, H, Hkv, D, prefix_k, prefix_v, P, pool_format, pool_k, pool_v, pool_ks, pool_vs,
                              pages_cols, lens, lens_stride, cur_k, cur_v, workspace, workspace_bytes, stream, ex);
}

// copies entries 0 .. n - 1 of row `origin` of a page table [rows, stride] to rows curr .. curr + forks - 1
__global__ __launch_bounds__(256) void page_fork_kernel(int32_t *table, long stride, int origin, int curr, int n) {
    const int32_t *src = table + (long)origin * stride;
    int32_t *dst = table + (long)(curr + blockIdx.y) * stride;
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = src[i];
}

extern "C" int smh_page_fork(int32_t *table, int rows, long stride, int origin, int curr, int forks, int n, smh_stream_t stream) {
    SMH_REQUIRE(table && rows > 0 && stride > 0 && n >= 0 && n <= stride, "smh_page_fork: table=%p rows=%d stride=%ld n=%d", (void *)table, rows, stride, n);
    SMH_REQUIRE(origin >= 0 && origin < rows && forks >= 0 && curr >= 0 && curr + forks <= rows && forks <= 65535,
                "smh_page_fork: origin=%d curr=%d forks=%d outside the table's %d rows", origin, curr, forks, rows);
    SMH_REQUIRE(origin < curr || origin >= curr + forks, "smh_page_fork: the origin row lies inside the rows it is copied to");
    if (forks == 0 || n == 0) return 0;
    hipLaunchKernelGGL(page_fork_kernel, dim3((unsigned)((n + 255) / 256), (unsigned)forks), dim3(256), 0, (hipStream_t)stream, table, stride, origin, curr, n);
    return smh::launch_status();
}

// ---- the same attention for callers that cannot allocate ---------------------------------------------------------
// The prefix partials of smh_shared_prefix_attn_static live in this array instead of a caller's workspace.  Every GPU
// the library runs on holds its own copy at its own address for the life of the process; host code never uses the
// array's name as an address, only what hipGetSymbolAddress returned for the current device.
constexpr size_t ATT_STATIC_SCRATCH_BYTES = (size_t)16 << 20;
static __device__ __align__(256) unsigned char scratch[ATT_STATIC_SCRATCH_BYTES];
constexpr int ATT_STATIC_MAX_DEVICES = 64;
static std::mutex g_scratch_mutex;
static void *g_scratch_ptr[ATT_STATIC_MAX_DEVICES] = {};

// Device address of `scratch` on the current device, looked up once per device.
static int static_scratch(void **ptr_out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) { smh::set_error("smh_shared_prefix_attn_static: hipGetDevice: %s", hipGetErrorString(e)); return (int)e; }
    if (dev < 0 || dev >= ATT_STATIC_MAX_DEVICES) { smh::set_error("smh_shared_prefix_attn_static: device %d outside [0,%d)", dev, ATT_STATIC_MAX_DEVICES); return -1; }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void *ptr = nullptr;
        e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr) {
            smh::set_error("smh_shared_prefix_attn_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
            return e != hipSuccess ? (int)e : -1;
        }
        g_scratch_ptr[dev] = ptr;
    }
    *ptr_out = g_scratch_ptr[dev];
    return 0;
}

extern "C" size_t smh_attn_static_scratch_bytes(void) { return ATT_STATIC_SCRATCH_BYTES; }

extern "C" int smh_shared_prefix_attn_static(const void *q, void *out, int B, int H, int Hkv, int D,
                                             const void *prefix_k, const void *prefix_v, int P,
                                             int suffix_format, const void *suffix_k, const void *suffix_v,
                                             const void *suffix_ks, const void *suffix_vs, int Smax,
                                             const int32_t *lens, int lens_stride, const void *cur_k, const void *cur_v,
                                             smh_stream_t stream) {
    using namespace smh;
    const char *who = "smh_shared_prefix_attn_static";
    // (every argument check comes before the scratch array's address is asked for: a refused call does not touch the device)
    SMH_REQUIRE(D == ATT_D, "%s: head dim %d (only 128)", who, D);
    SMH_REQUIRE(B >= 0 && B <= 65535 && H > 0 && Hkv > 0 && H % Hkv == 0 && P >= 0, "%s: B=%d (at most 65535) H=%d Hkv=%d P=%d", who, B, H, Hkv, P);
    // the partials the two launches exchange: one (max, sum, o[128]) per prefix slice and query, as smh_shared_prefix_attn plans them
    int tw = ATT_TW_MAX, qgroups = 1;
    attn_plan(P, Hkv, B * (H / Hkv), &tw, &qgroups);
    const size_t splits = P > 0 ? (size_t)(P + tw - 1) / tw : 0;
    const size_t need = splits * (size_t)B * H * (ATT_D + 2) * sizeof(float);
    SMH_REQUIRE(need <= ATT_STATIC_SCRATCH_BYTES, "%s: B=%d H=%d P=%d needs %zu bytes of scratch, the static array holds %zu (use smh_shared_prefix_attn with a workspace)",
                who, B, H, P, need, ATT_STATIC_SCRATCH_BYTES);
    SMH_REQUIRE(B == 0 || (q && out), "%s: null q/out", who);
    SMH_REQUIRE(P == 0 || (prefix_k && prefix_v), "%s: null prefix", who);
    SMH_REQUIRE(suffix_format == SMH_KV_NONE || (suffix_k && suffix_v && lens && Smax > 0), "%s: suffix arguments incomplete", who);
    if (B == 0) return 0;
    void *ws = nullptr;
    const int st = static_scratch(&ws);
    if (st) return st;
    return shared_prefix_attn(who, false, q, out, B, H, Hkv, D, prefix_k, prefix_v, P, suffix_format, suffix_k, suffix_v, suffix_ks, suffix_vs,
                              Smax, lens, lens_stride, cur_k, cur_v, ws, ATT_STATIC_SCRATCH_BYTES, stream);
}

extern "C" int smh_shared_prefix_attn_one(const void *q, void *out, int B, int H, int Hkv, int D,
                                          const void *prefix_k, const void *prefix_v, int P,
                                          int suffix_format, const void *suffix_k, const void *suffix_v,
                                          const void *suffix_ks, const void *suffix_vs, int Smax,
                                          const int32_t *lens, int lens_stride, const void *cur_k, const void *cur_v,
                                          void *workspace, size_t workspace_bytes, smh_stream_t stream) {
    return shared_prefix_attn("smh_shared_prefix_attn_one", true, q, out, B, H, Hkv, D, prefix_k, prefix_v, P, suffix_format, suffix_k,
                              suffix_v, suffix_ks, suffix_vs, Smax, lens, lens_stride, cur_k, cur_v, workspace, workspace_bytes, stream);
}


extern "C" size_t smh_attn_qkv_workspace_bytes(int B, int H, int P) {
    if (B <= 0 || H <= 0) return ATT_COUNTER_BYTES + 256;
    size_t splits = (size_t)(P > 0 ? (P + 31) / 32 : 0) + 1;      // worst case: 32 rows per workgroup; + the suffix partial
    return ATT_COUNTER_BYTES + splits * (size_t)B * (size_t)H * (smh::ATT_D + 2) * sizeof(float) + 256;
}

extern "C" int smh_shared_prefix_attn_qkv(const void *qkv_partial, int ksplit, void *out, int B, int H, int Hkv, int D,
                                          const void *cos_tab, const void *sin_tab, const int32_t *pos_dev,
                                          const void *prefix_k, const void *prefix_v, int P,
                                          void *cache_k, void *cache_ks, void *cache_v, void *cache_vs, int Smax,
                                          const int32_t *t_dev, const int32_t *pages, int pages_stride, int single_launch,
                                          void *workspace, size_t workspace_bytes, smh_stream_t stream) {
    using namespace smh;
    const char *who = "smh_shared_prefix_attn_qkv";
    SMH_REQUIRE(pages == nullptr || pages_stride >= Smax, "%s: pages_stride=%d must cover the %d rows of a branch", who, pages_stride, Smax);
    SMH_REQUIRE(D == ATT_D, "%s: head dim %d (only 128)", who, D);
    SMH_REQUIRE(B >= 0 && B <= 16 && H > 0 && Hkv > 0 && H % Hkv == 0 && P >= 0, "%s: B=%d (at most 16) H=%d Hkv=%d P=%d", who, B, H, Hkv, P);
    SMH_REQUIRE(ksplit >= 1 && ksplit <= 16, "%s: ksplit=%d", who, ksplit);
    SMH_REQUIRE(B * (H / Hkv) <= ATT_FUSED_MAX_Q, "%s: %d queries per kv head (at most %d)", who, B * (H / Hkv), ATT_FUSED_MAX_Q);
    if (B == 0) return 0;
    SMH_REQUIRE(qkv_partial && out && cos_tab && sin_tab && pos_dev, "%s: null pointer", who);
    SMH_REQUIRE(P == 0 || (prefix_k && prefix_v), "%s: null prefix", who);
    SMH_REQUIRE(cache_k && cache_ks && cache_v && cache_vs && t_dev && Smax > 0, "%s: the suffix cache and its row counter are required", who);
    AttnParams p{};
    p.out = (half_t *)out;
    p.prefix_k = (const half_t *)prefix_k; p.prefix_v = (const half_t *)prefix_v;
    p.suffix_k = cache_k; p.suffix_v = cache_v;
    p.suffix_ks = (const half_t *)cache_ks; p.suffix_vs = (const half_t *)cache_vs;
    p.lens = t_dev; p.lens_stride = 0;
    p.suffix_batch_stride_rows = Smax;
    p.pages = pages; p.pages_stride = pages_stride; p.page_bytes = 4; p.pool_rows = (long)B * Smax;   // a branch reads its own rows and its ancestors', all below B
    p.pfx_row_stride = (long)Hkv * ATT_D; p.pfx_head_stride = ATT_D;
    p.sfx_row_stride = (long)Hkv * ATT_D; p.sfx_head_stride = ATT_D;
    p.B = B; p.H = H; p.Hkv = Hkv; p.n_rep = H / Hkv; p.Bq = B * p.n_rep;
    p.P = P; p.suffix_format = SMH_KV_Q40; p.causal = 0;
    p.scale_log2 = LOG2E / sqrtf((float)D);
    int qgroups = 1;
    if (single_launch) p.tw = min(attn_plan_tw(P, Hkv), ATT_ONE_TW);
    else attn_plan(P, Hkv, p.Bq, &p.tw, &qgroups);
    p.splits = P > 0 ? (P + p.tw - 1) / p.tw : 0;
    p.qkv = (const float *)qkv_partial; p.qkv_ks = ksplit;
    p.cos_tab = (const half_t *)cos_tab; p.sin_tab = (const half_t *)sin_tab; p.pos_dev = pos_dev;
    p.app_k = (uint8_t *)cache_k; p.app_v = (uint8_t *)cache_v;
    p.app_ks = (half_t *)cache_ks; p.app_vs = (half_t *)cache_vs;
    p.app_t = t_dev; p.app_smax = Smax;
    if (single_launch) {
        p.suffix_waves = attn_plan_suffix_waves(p.splits, p.Bq, Hkv);
        // workspace = [arrival counters | partials of splits + 1 passes]
        SMH_REQUIRE((size_t)Hkv * ((p.Bq + 15) / 16) * sizeof(uint32_t) <= ATT_COUNTER_BYTES, "%s: %d kv heads x %d query tiles", who, Hkv, (p.Bq + 15) / 16);
        size_t n_part = (size_t)(p.splits + 1) * Hkv * p.Bq;
        size_t need = ATT_COUNTER_BYTES + n_part * (ATT_D + 2) * sizeof(float);
        SMH_REQUIRE(workspace && workspace_bytes >= need, "%s: workspace %zu < %zu bytes", who, workspace_bytes, need);
        p.counters = (uint32_t *)workspace;
        p.part_o = (float *)((char *)workspace + ATT_COUNTER_BYTES);
        p.part_ml = p.part_o + n_part * ATT_D;
        hipLaunchKernelGGL(attn_one_kernel<true>, dim3(p.splits + (p.Bq + 4 / p.suffix_waves - 1) / (4 / p.suffix_waves), Hkv), dim3(256), 0, (hipStream_t)stream, p);
        return launch_status();
    }
    size_t n_part = (size_t)p.splits * Hkv * p.Bq;
    SMH_REQUIRE(p.splits == 0 || (workspace && workspace_bytes >= n_part * (ATT_D + 2) * sizeof(float)),
                "%s: workspace %zu < %zu bytes", who, workspace_bytes, n_part * (ATT_D + 2) * sizeof(float));
    p.part_o = (float *)workspace;
    p.part_ml = p.part_o + n_part * ATT_D;
    if (p.splits > 0)
        hipLaunchKernelGGL(attn_prefix_kernel<true>, dim3(p.splits, Hkv, qgroups), dim3(256), 0, (hipStream_t)stream, p);
    p.suffix_waves = attn_plan_suffix_waves_two((long)B * H);
    hipLaunchKernelGGL(attn_suffix_kernel<true>, dim3((unsigned)(((H * p.suffix_waves + 3) / 4) * ((B + 7) / 8 * 8))), dim3(256), 0, (hipStream_t)stream, p);
    return launch_status();
}

// Causal prefill attention, expressed as the suffix kernel with "branch" = query position:
// query s attends to rows 0..s of the same K/V tensors (batch stride 0, no shared prefix).
extern "C" int smh_prefill_attn(const void *q, const void *k, const void *v, void *out, int S, int H, int Hkv,
                                int D, smh_stream_t stream) {
    using namespace smh;
    SMH_REQUIRE(D == ATT_D, "smh_prefill_attn: head dim %d (only 128)", D);
    SMH_REQUIRE(S >= 0 && H > 0 && Hkv > 0 && H % Hkv == 0, "smh_prefill_attn: S=%d H=%d Hkv=%d", S, H, Hkv);
    if (S == 0) return 0;
    SMH_REQUIRE(q && k && v && out, "smh_prefill_attn: null pointer");
    PrefillParams p;
    p.q = (const half_t *)q; p.k = (const half_t *)k; p.v = (const half_t *)v; p.out = (half_t *)out;
    p.S = S; p.H = H; p.Hkv = Hkv; p.n_rep = H / Hkv;
    p.scale_log2 = LOG2E / sqrtf((float)D);
    hipLaunchKernelGGL(attn_prefill_kernel, dim3((unsigned)((S + 63) / 64), (unsigned)H), dim3(256), 0, (hipStream_t)stream, p);
    return launch_status();
}
