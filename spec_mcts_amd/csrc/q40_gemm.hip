// Q4_0 dequant + matmul for large batches (decode at B = 100, prefill): c[M,N] = a[M,K] . deq(W)[K,N].
//
// A workgroup owns 128 rows of A, one 128-column block of the weight (one 64-byte packed row per
// k) and a slice of K.  Per 32-row step
//   * the 128 x 32 tile of A is staged in LDS (double buffered, one barrier per step; row pitch 40
//     halves, so the 16 rows read by one ds_read_b128 pass fall on distinct banks);
//   * every wave loads the step's 8 weight dwords per lane, but decodes only ONE byte position
//     (wave w <-> byte w of each dword): 32 of the block's 128 columns.  Decoding is the same
//     perm / and-or / packed-fp16 sequence as the GEMV and lands directly in the B-operand layout
//     of v_mfma_f32_16x16x32_f16, so dequantised weights never travel through LDS or HBM;
//   * the wave multiplies its two B operands with all (up to 8) 16-row tiles of A;
//   * the next step's weights and A rows are already in flight while this step is computed.
// K-slices are written as fp32 slabs and added by the consuming kernel, as for the GEMV.
//
// At M = 100 the work sits on the ridge of the roofline: 2*M*N*K flops against
// N*K*0.53125 + 2*M*(K+N) bytes.
#include "q40_matmul.hpp"

namespace smh {

constexpr int GEMM_BM = 128;
constexpr int GEMM_THREADS = 256;
constexpr int GEMM_PITCH = 40;             // halves per LDS row of the A tile

struct GemmRegs {
    uint32_t wv[8], sv[8];
    u32x4 a0, a1;
};

__global__ __launch_bounds__(GEMM_THREADS) void q40_gemm_kernel(MatmulParams p) {
    __shared__ __attribute__((aligned(16))) half_t a_tile[2][GEMM_BM][GEMM_PITCH];

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int c = lane & 15;
    const int g = lane >> 4;
    int bid = blockIdx.x;
    const int unit = bid % p.units;  bid /= p.units;
    const int mb = bid % p.mblocks;
    const int slice = bid / p.mblocks;
    int sg = 0;
    if (p.nseg > 1 && unit >= p.seg[1].unit0) sg = 1;
    if (p.nseg > 2 && unit >= p.seg[2].unit0) sg = 2;
    const MatmulSegment seg = p.seg[sg];
    const int block = unit - seg.unit0;
    const int m0 = mb * GEMM_BM;
    const int m_count = min(GEMM_BM, p.M - m0);
    const int tiles = (m_count + 15) / 16;

    const long w_row = seg.N / 2;
    const long s_row = seg.N / 64;
    const uint8_t *wp = seg.w + (long)block * 64 + 4 * c;
    const half_t *sp = seg.s + (long)block * 2;
    const uint32_t sel = 0x0c000c00u | (uint32_t)wave | ((uint32_t)(4 + wave) << 16);

    // staging role: thread t copies 16 halves of row t/2
    const int st_row = tid >> 1;
    const int st_col = (tid & 1) * 16;
    const half_t *st_src = p.a + (long)min(m0 + st_row, p.M - 1) * p.lda + st_col;

    f4 acc[2][8];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int t = 0; t < 8; ++t) acc[h][t] = f4{0.f, 0.f, 0.f, 0.f};

    const int step0 = slice * p.steps_per_slice;
    const int step1 = min(step0 + p.steps_per_slice, (p.K + 31) / 32);

    auto load_step = [&](GemmRegs &r, int step) {
        const int kb = step * 32;
        r.a0 = u32x4{0, 0, 0, 0};
        r.a1 = u32x4{0, 0, 0, 0};
        if (kb + st_col < p.K) r.a0 = *reinterpret_cast<const u32x4 *>(st_src + kb);
        if (kb + st_col + 8 < p.K) r.a1 = *reinterpret_cast<const u32x4 *>(st_src + kb + 8);
        const int k0 = kb + 8 * g;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int k = min(k0 + i, p.K - 1);
            r.wv[i] = *reinterpret_cast<const uint32_t *>(wp + (long)k * w_row);
            r.sv[i] = *reinterpret_cast<const uint32_t *>(sp + (long)k * s_row);
        }
    };

    GemmRegs cur, nxt;
    if (step0 < step1) load_step(cur, step0);
    int buf = 0;
    for (int step = step0; step < step1; ++step) {
        *reinterpret_cast<u32x4 *>(&a_tile[buf][st_row][st_col]) = cur.a0;
        *reinterpret_cast<u32x4 *>(&a_tile[buf][st_row][st_col + 8]) = cur.a1;
        if (step + 1 < step1) load_step(nxt, step + 1);
        // ---- decode this wave's byte position ----
        h2 bh[4], bl[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint32_t pr = __builtin_amdgcn_perm(cur.wv[2 * j + 1], cur.wv[2 * j], sel) ^ (NIBBLE_FLIP & 0x00FF00FFu);
            bh[j] = codes_high(pr) * as_h2(pack_lo16(cur.sv[2 * j], cur.sv[2 * j + 1]));
            bl[j] = codes_low(pr) * as_h2(pack_hi16(cur.sv[2 * j], cur.sv[2 * j + 1]));
        }
        h8 vb_h = {bh[0].x, bh[0].y, bh[1].x, bh[1].y, bh[2].x, bh[2].y, bh[3].x, bh[3].y};
        h8 vb_l = {bl[0].x, bl[0].y, bl[1].x, bl[1].y, bl[2].x, bl[2].y, bl[3].x, bl[3].y};
        __syncthreads();                    // a_tile[buf] holds this step; the other buffer is free again
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            if (t < tiles) {
                h8 av = *reinterpret_cast<const h8 *>(&a_tile[buf][t * 16 + c][8 * g]);
                acc[0][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, vb_h, acc[0][t], 0, 0, 0);
                acc[1][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, vb_l, acc[1][t], 0, 0, 0);
            }
        }
        cur = nxt;
        buf ^= 1;
    }

    // accumulator element r of acc[h][t] is row m0 + 16t + 4g + r, column 128*block + 64h + 4c + wave
    const int n_base = seg.col0 + block * 128 + 4 * c + wave;
    float *slab = p.partial + (long)slice * p.M * p.n_total;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int t = 0; t < 8; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = m0 + 16 * t + 4 * g + r;
                const int n = n_base + 64 * h;
                if (m < p.M) {
                    if (p.direct) p.c[(long)m * p.ldc + n] = matmul_epilogue(p, acc[h][t][r], m, n);
                    else slab[(long)m * p.n_total + n] = acc[h][t][r];
                }
            }
}

void gemm_fill_plan(MatmulParams &p) {
    int unit0 = 0, col0 = 0;
    for (int i = 0; i < p.nseg; ++i) {
        p.seg[i].unit0 = unit0;
        p.seg[i].col0 = col0;
        unit0 += p.seg[i].N / 128;
        col0 += p.seg[i].N;
    }
    p.units = unit0;
    p.units_pad = unit0;
    p.n_total = col0;
    p.mblocks = (p.M + GEMM_BM - 1) / GEMM_BM;
    const int steps = (p.K + 31) / 32;
    const long tiles = (long)p.units * p.mblocks;
    static const int target = env_int("SMH_GEMM_WGS", 512);
    int ks = (int)(target / tiles);
    if (ks < 1) ks = 1;
    if (ks > steps / 4) ks = steps / 4 > 0 ? steps / 4 : 1;
    if (ks > SMH_MAX_KSPLIT) ks = SMH_MAX_KSPLIT;
    p.steps_per_slice = (steps + ks - 1) / ks;
    p.ksplit = (steps + p.steps_per_slice - 1) / p.steps_per_slice;
}

int gemm_launch(const MatmulParams &p, hipStream_t stream) {
    dim3 grid((unsigned)((long)p.units * p.mblocks * p.ksplit));
    hipLaunchKernelGGL(q40_gemm_kernel, grid, dim3(GEMM_THREADS), 0, stream, p);
    return launch_status();
}

}  // namespace smh
