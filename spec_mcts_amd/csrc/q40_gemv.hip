// Q4_0 dequant + matmul for small batches (M <= 16): c[M,N] = a[M,K] . deq(W)[K,N].
//
// The weight is streamed exactly once, in its checkpoint layout (bytes [K, N/2], scales
// [K, N/64]); the kernel is bound by HBM bandwidth.  Algorithmic traffic per launch:
// N*K/2 + 2*N*K/64 + 2*M*K + 2*M*N bytes.
//
// Work decomposition
//   * a workgroup owns TWO adjacent 128-column blocks (one full 128-byte line of packed nibbles
//     per k, so no cache line is shared with another workgroup) and a slice of K; its waves take
//     alternate pairs of 32-row steps of that slice and issue the loads of both steps of a pair
//     before decoding either;
//   * inside a step, lane l = 16*g + c loads the 8 bytes at offset 8c of rows k0 + 8g .. k0 + 8g + 7,
//     i.e. 8 k-values of 16 columns.  Byte-permutes pair the same nibble of two consecutive rows,
//     one AND-OR drops the pair into the mantissa of fp16 1024.0, one packed fp16 op recovers the
//     exact integer code and one packed multiply applies the per-row scales -> the fp16 value the
//     reference dequantiser produces, already in the register layout of the B operand of
//     v_mfma_f32_16x16x32_f16 (lane = column, 8 consecutive k per lane).  The reduction over the
//     lanes' k-groups happens inside the matrix core; rows of A are the (up to 16) batch rows.
//   * partial sums of the waves are added through LDS and written, one fp32 [M, N] slab per
//     K-slice, with plain coalesced stores.  Nothing waits for another workgroup: the slabs are
//     added, in slice order (so results do not depend on scheduling), by whichever kernel consumes
//     the product (partial_ops.hip: plain reduce, residual + RMSNorm, RoPE + KV append, SiLU*up).
//   * up to three weights that share the input (wq|wk|wv, w1|w3) run as segments of one launch.
//
// blockIdx.x = slice * pairs_pad + pair with pairs_pad a multiple of 8: workgroups are dealt
// round-robin to the 8 XCDs, so all K-slices of a column pair run behind the same L2.
#include <stdlib.h>

#include "q40_matmul.hpp"

namespace smh {

constexpr int GEMV_COLS = 256;             // columns per workgroup

// registers of one 32-row step of one lane
struct GemvStep {
    u32x2 wv[8];     // 8 bytes of 8 consecutive rows
    uint32_t sv[8];  // (scale of columns 0..63, scale of columns 64..127) of this lane's block, per row
    h8 av;           // 8 activations of batch row c
};

__device__ __forceinline__ void gemv_load(GemvStep &st, int K, const uint8_t *wp, const half_t *sp,
                                          const half_t *ap, long w_row, long s_row, int k0) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int k = min(k0 + i, K - 1);
        st.wv[i] = *reinterpret_cast<const u32x2 *>(wp + (long)k * w_row);
        st.sv[i] = *reinterpret_cast<const uint32_t *>(sp + (long)k * s_row);
    }
    if (k0 < K) {
        st.av = *reinterpret_cast<const h8 *>(ap + k0);
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) st.av[i] = (half_t)0.f;
    }
}

// acc[d][h][b]: dword d of the lane's 8 bytes, nibble half h (0 = high = columns 0..63 of the block),
// byte b of the dword
__device__ __forceinline__ void gemv_compute(const GemvStep &st, f4 (&acc)[2][2][4]) {
    h2 s_hi[4], s_lo[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        s_hi[j] = as_h2(pack_lo16(st.sv[2 * j], st.sv[2 * j + 1]));
        s_lo[j] = as_h2(pack_hi16(st.sv[2 * j], st.sv[2 * j + 1]));
    }
#pragma unroll
    for (int d = 0; d < 2; ++d) {
        uint32_t u[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) u[i] = st.wv[i][d] ^ NIBBLE_FLIP;
#define SMH_GEMV_BYTE(B)                                                                        \
        {                                                                                       \
            h2 bh[4], bl[4];                                                                    \
            _Pragma("unroll") for (int j = 0; j < 4; ++j) {                                     \
                uint32_t pr = pair_bytes<B>(u[2 * j], u[2 * j + 1]);                            \
                bh[j] = codes_high(pr) * s_hi[j];                                               \
                bl[j] = codes_low(pr) * s_lo[j];                                                \
            }                                                                                   \
            h8 vb_h = {bh[0].x, bh[0].y, bh[1].x, bh[1].y, bh[2].x, bh[2].y, bh[3].x, bh[3].y}; \
            h8 vb_l = {bl[0].x, bl[0].y, bl[1].x, bl[1].y, bl[2].x, bl[2].y, bl[3].x, bl[3].y}; \
            acc[d][0][B] = __builtin_amdgcn_mfma_f32_16x16x32_f16(st.av, vb_h, acc[d][0][B], 0, 0, 0); \
            acc[d][1][B] = __builtin_amdgcn_mfma_f32_16x16x32_f16(st.av, vb_l, acc[d][1][B], 0, 0, 0); \
        }
        SMH_GEMV_BYTE(0)
        SMH_GEMV_BYTE(1)
        SMH_GEMV_BYTE(2)
        SMH_GEMV_BYTE(3)
#undef SMH_GEMV_BYTE
    }
}

template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) void q40_gemv_kernel(MatmulParams p) {
    extern __shared__ float red[];          // [WAVES][M][256]
    constexpr int THREADS = WAVES * 64;

    const int unit = blockIdx.x % p.units_pad;
    const int slice = blockIdx.x / p.units_pad;
    if (unit >= p.units) return;
    // which segment (weight) does this column pair belong to
    int sg = 0;
    if (p.nseg > 1 && unit >= p.seg[1].unit0) sg = 1;
    if (p.nseg > 2 && unit >= p.seg[2].unit0) sg = 2;
    const MatmulSegment seg = p.seg[sg];
    const int pair = unit - seg.unit0;

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int c = lane & 15;
    const int g = lane >> 4;

    const long w_row = seg.N / 2;          // bytes per k
    const long s_row = seg.N / 64;         // scales per k
    const int col0 = pair * GEMV_COLS;     // first column (inside the segment) of this workgroup
    // lanes c >= 8 belong to the second block of the pair; when N/128 is odd the last pair has none:
    // such lanes re-read the first block (valid memory) and their results are dropped
    const bool has_block = col0 + 128 * (c >> 3) < seg.N;
    const int c_ld = has_block ? c : (c & 7);
    const uint8_t *wp = seg.w + (long)pair * 128 + 8 * c_ld;
    const half_t *sp = seg.s + (long)pair * 4 + 2 * (c_ld >> 3);
    const int m_a = min(c, p.M - 1);       // row of A this lane feeds (rows >= M are never stored)
    const half_t *ap = p.a + (long)m_a * p.lda;

    f4 acc[2][2][4];
#pragma unroll
    for (int d = 0; d < 2; ++d)
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int b = 0; b < 4; ++b) acc[d][h][b] = f4{0.f, 0.f, 0.f, 0.f};

    const int step0 = slice * p.steps_per_slice;
    const int step1 = min(step0 + p.steps_per_slice, (p.K + 31) / 32);
    for (int step = step0 + 2 * wave; step < step1; step += 2 * WAVES) {
        GemvStep s0, s1;
        gemv_load(s0, p.K, wp, sp, ap, w_row, s_row, step * 32 + 8 * g);
        const bool two = step + 1 < step1;
        if (two) gemv_load(s1, p.K, wp, sp, ap, w_row, s_row, (step + 1) * 32 + 8 * g);
        gemv_compute(s0, acc);
        if (two) gemv_compute(s1, acc);
    }

    // ---- add the waves' partial sums through LDS ----
    // accumulator element r of acc[d][h][b] in lane (g, c) is row m = 4g + r,
    // column 128*(c>>3) + 64h + 8*(c&7) + 4d + b of the workgroup's 256
    const int col_lane = 128 * (c >> 3) + 8 * (c & 7);
#pragma unroll
    for (int d = 0; d < 2; ++d)
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int b = 0; b < 4; ++b)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int m = 4 * g + r;
                    if (m < p.M) red[(wave * p.M + m) * GEMV_COLS + col_lane + 64 * h + 4 * d + b] = acc[d][h][b][r];
                }
    __syncthreads();

    // thread -> outputs idx = tid, tid + THREADS, ... with idx = m * 256 + local column
    const int outputs = p.M * GEMV_COLS;
    float *slab = p.partial + (long)slice * p.M * p.n_total;
    for (int idx = tid; idx < outputs; idx += THREADS) {
        float sum = 0.f;
#pragma unroll
        for (int wv_ = 0; wv_ < WAVES; ++wv_) sum += red[wv_ * outputs + idx];
        const int m = idx >> 8, n_seg = col0 + (idx & 255);
        if (n_seg >= seg.N) continue;
        const int n = seg.col0 + n_seg;
        if (p.direct) p.c[(long)m * p.ldc + n] = matmul_epilogue(p, sum, m, n);
        else slab[(long)m * p.n_total + n] = sum;
    }
}

}  // namespace smh

namespace smh {

int env_int(const char *name, int dflt) {
    const char *v = getenv(name);
    return v ? atoi(v) : dflt;
}

// K is cut into at most SMH_MAX_KSPLIT slices so that about `target` workgroups are in flight
// (256 CUs) while every wave still has a pair of steps to do.
void gemv_plan(int n_total_units, int K, int waves, int *ksplit, int *steps_per_slice) {
    const int steps = (K + 31) / 32;
    static const int target_wgs = env_int("SMH_GEMV_WGS", 512);
    const int unit = 2 * waves;
    int want = (target_wgs + n_total_units - 1) / n_total_units;
    int max_split = (steps + unit - 1) / unit;
    int ks = want < 1 ? 1 : want;
    if (ks > max_split) ks = max_split;
    if (ks > SMH_MAX_KSPLIT) ks = SMH_MAX_KSPLIT;
    int sps = (steps + ks - 1) / ks;
    sps = (sps + unit - 1) / unit * unit;
    ks = (steps + sps - 1) / sps;
    *ksplit = ks;
    *steps_per_slice = sps;
}

int gemv_waves(int M) {
    static const int waves_pref = env_int("SMH_GEMV_WAVES", 4);
    int waves = waves_pref;
    while (waves > 2 && (size_t)waves * M * GEMV_COLS * sizeof(float) > 48 * 1024) waves >>= 1;   // LDS budget
    return waves;
}

void gemv_fill_plan(MatmulParams &p) {
    int unit0 = 0, col0 = 0;
    for (int i = 0; i < p.nseg; ++i) {
        p.seg[i].unit0 = unit0;
        p.seg[i].col0 = col0;
        unit0 += (p.seg[i].N + GEMV_COLS - 1) / GEMV_COLS;
        col0 += p.seg[i].N;
    }
    p.units = unit0;
    p.units_pad = (unit0 + 7) / 8 * 8;
    p.n_total = col0;
    gemv_plan(p.units, p.K, gemv_waves(p.M), &p.ksplit, &p.steps_per_slice);
}

int gemv_launch(const MatmulParams &p, hipStream_t stream) {
    const int waves = gemv_waves(p.M);
    dim3 grid((unsigned)(p.units_pad * p.ksplit));
    size_t lds = (size_t)waves * p.M * GEMV_COLS * sizeof(float);
    if (waves == 2) hipLaunchKernelGGL(q40_gemv_kernel<2>, grid, dim3(128), lds, stream, p);
    else if (waves == 8) hipLaunchKernelGGL(q40_gemv_kernel<8>, grid, dim3(512), lds, stream, p);
    else hipLaunchKernelGGL(q40_gemv_kernel<4>, grid, dim3(256), lds, stream, p);
    return launch_status();
}

}  // namespace smh
