// Q4_0 dequant + matmul for large batches (decode at B = 100, prefill): c[M,N] = a[M,K] . deq(W)[K,N].
//
// A workgroup of 8 waves owns 128 rows of A, two adjacent 128-column blocks of the weight (one full
// 128-byte line of packed nibbles per k) and a slice of K.  Everything a 32-row step needs - 4 KB of
// nibbles, 256 B of scales, the 128 x 32 tile of A - goes global -> LDS by DMA (global_load_lds) into a
// 4-stage ring shared by the workgroup, three steps ahead of the step being computed; one barrier per
// step both publishes a stage and frees the oldest one.
//   * wave w decodes ONE byte position of ONE block (block w/4, byte w%4 of every dword): perm pairs
//     the byte of two consecutive rows, and-or drops the nibbles into fp16 mantissas, one packed op
//     recovers the exact code and one packed multiply applies the scales - the value the reference's
//     dequantiser produces, born in the B-operand layout of v_mfma_f32_16x16x32_f16, so dequantised
//     weights never travel through LDS or HBM;
//   * it multiplies its two B operands (high / low nibbles = columns c and c+64) with all (up to 8)
//     16-row tiles of A, read from LDS with an XOR swizzle that keeps ds_read_b128 conflict-free;
//   * the accumulators leave through LDS one row tile at a time, so global stores are 32-byte
//     contiguous per lane; K-slices are written as fp32 slabs and added by the consuming kernel.
//
// At M = 100 the work sits on the ridge of the roofline: 2*M*N*K flops against
// N*K*0.53125 + 2*M*(K+N) bytes.
#include "q40_matmul.hpp"

namespace smh {

constexpr int GEMM_BM = 128;
constexpr int GEMM_WAVES = 8;
constexpr int GEMM_THREADS = GEMM_WAVES * 64;
constexpr int GEMM_STAGES = 4;
constexpr int GS_W = 32 * 128;                 // nibbles
constexpr int GS_S = 32 * 8;                   // scales
constexpr int GS_A = GEMM_BM * 64;             // A tile, 64 B per row, 16-byte chunks XOR-swizzled
constexpr int GS_PAD = 256;                    // landing zone of the padding DMA (keeps 2 DMAs per wave per stage)
constexpr int GS_BYTES = GS_W + GS_S + GS_A + GS_PAD;      // 12800
constexpr int GEMM_LDS = GEMM_STAGES * GS_BYTES;           // 51200
constexpr int GEMM_COLS = 256;

typedef const __attribute__((address_space(1))) void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;

__global__ __launch_bounds__(GEMM_THREADS) void q40_gemm_kernel(MatmulParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int c = lane & 15;
    const int g = lane >> 4;
    int bid = blockIdx.x;
    // slot -> unit: each XCD (blockIdx % 8) takes a contiguous run of column units, which share scale lines
    const int slot = bid % p.units_pad;  bid /= p.units_pad;
    const int unit = (slot & 7) * (p.units_pad >> 3) + (slot >> 3);
    if (unit >= p.units) return;
    const int mb = bid % p.mblocks;
    const int slice = bid / p.mblocks;
    int sg = 0;
    if (p.nseg > 1 && unit >= p.seg[1].unit0) sg = 1;
    if (p.nseg > 2 && unit >= p.seg[2].unit0) sg = 2;
    const MatmulSegment seg = p.seg[sg];
    const int pair = unit - seg.unit0;
    const int col0 = pair * GEMM_COLS;
    const bool two_blocks = col0 + 128 < seg.N;
    const int m0 = mb * GEMM_BM;
    const int m_count = min(GEMM_BM, p.M - m0);
    const int tiles = (m_count + 15) / 16;
    const int blk = wave >> 2;                 // block of the pair this wave decodes
    const uint32_t sel = 0x0c000c00u | (uint32_t)(wave & 3) | ((uint32_t)(4 + (wave & 3)) << 16);

    const long w_row = seg.N / 2;
    const long s_row = seg.N / 64;
    // ---- this wave's two DMA instructions per stage ----
    //  first : waves 0..3 -> 8 rows of nibbles each; wave 4 -> scales; waves 5..7 -> padding (scales again)
    //  second: wave w -> rows 16w .. 16w+15 of the A tile
    const uint8_t *w_lane = seg.w + (long)pair * 128 + 16 * (two_blocks ? (lane & 7) : (lane & 3));
    const half_t *s_lane = seg.s + (long)pair * 4 + 2 * (two_blocks ? (lane & 1) : 0);
    const int a_row = 16 * wave + (lane >> 2);                            // row of the tile this lane fetches
    const int a_chunk = (lane & 3) ^ ((a_row >> 2) & 3);                  // logical 16-byte chunk stored in slot lane&3
    const half_t *a_lane = p.a + (long)min(m0 + a_row, p.M - 1) * p.lda;

    auto issue = [&](int step, int stage) {
        uint8_t *st = lds + stage * GS_BYTES;
        const int k0 = step * 32;
        if (wave < 4) {
            const int row = min(k0 + 8 * wave + (lane >> 3), p.K - 1);
            __builtin_amdgcn_global_load_lds((gptr_t)(w_lane + (long)row * w_row), (lptr_t)(st + wave * 1024), 16, 0, 0);
        } else {
            const int row = min(k0 + (lane >> 1), p.K - 1);
            uint8_t *dst = (wave == 4) ? st + GS_W : st + GS_W + GS_S + GS_A;
            __builtin_amdgcn_global_load_lds((gptr_t)(s_lane + (long)row * s_row), (lptr_t)dst, 4, 0, 0);
        }
        const int col = min(k0 + 8 * a_chunk, p.K - 8);
        __builtin_amdgcn_global_load_lds((gptr_t)(a_lane + col), (lptr_t)(st + GS_W + GS_S + wave * 1024), 16, 0, 0);
    };

    f4 acc[2][8];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int t = 0; t < 8; ++t) acc[h][t] = f4{0.f, 0.f, 0.f, 0.f};

    const int step0 = slice * p.steps_per_slice;
    const int step1 = min(step0 + p.steps_per_slice, (p.K + 31) / 32);
    const int n_steps = max(step1 - step0, 0);
    // workgroups that share a K-slice read the same A tiles; each starts at a different step of the
    // slice (and wraps) so that they do not all pull the same L2 lines at the same time
    const int rot = n_steps > 0 ? (unit * 5) % n_steps : 0;
    auto step_of = [&](int i) { const int j = i + rot; return step0 + (j >= n_steps ? j - n_steps : j); };
#pragma unroll
    for (int i = 0; i < GEMM_STAGES - 1; ++i)
        if (i < n_steps) issue(step_of(i), i);

    for (int i = 0; i < n_steps; ++i) {
        const int later = min(GEMM_STAGES - 2, n_steps - 1 - i);     // younger steps this wave has in flight
        if (later >= 2) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
        else if (later == 1) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();     // stage i is complete for everyone; everyone is done with stage i-1
        if (i + GEMM_STAGES - 1 < n_steps) issue(step_of(i + GEMM_STAGES - 1), (i + GEMM_STAGES - 1) % GEMM_STAGES);

        const uint8_t *st = lds + (i % GEMM_STAGES) * GS_BYTES;
        const int k0 = step_of(i) * 32;
        // ---- decode this wave's byte position: exact fp16 code * scale ----
        uint32_t wv[8], sv[8];
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            wv[r] = *reinterpret_cast<const uint32_t *>(st + (8 * g + r) * 128 + 64 * blk + 4 * c);
            sv[r] = *reinterpret_cast<const uint32_t *>(st + GS_W + (8 * g + r) * 8 + 4 * blk);
        }
        u32x4 vh, vl;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t pr = __builtin_amdgcn_perm(wv[2 * j + 1], wv[2 * j], sel) ^ 0x00880088u;
            vh[j] = as_u32(codes_high(pr) * as_h2(pack_lo16(sv[2 * j], sv[2 * j + 1])));
            vl[j] = as_u32(codes_low(pr) * as_h2(pack_hi16(sv[2 * j], sv[2 * j + 1])));
        }
        const h8 vb_h = __builtin_bit_cast(h8, vh), vb_l = __builtin_bit_cast(h8, vl);
        const bool k_tail = k0 + 8 * g >= p.K;                       // only in the last step when K % 32 != 0
        const uint8_t *at = st + GS_W + GS_S;
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            if (t < tiles) {
                const int r = 16 * t + c;
                h8 av = *reinterpret_cast<const h8 *>(at + r * 64 + ((g ^ ((r >> 2) & 3)) << 4));
                if (k_tail) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) av[e] = (half_t)0.f;
                }
                acc[0][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, vb_h, acc[0][t], 0, 0, 0);
                acc[1][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, vb_l, acc[1][t], 0, 0, 0);
            }
        }
    }

    // ---- results leave one 16-row tile at a time through LDS: [16][256 + 4] floats ----
    // accumulator element r of acc[h][t] is row 16t + 4g + r, column 128*blk + 64h + 4c + (wave & 3)
    constexpr int OP = GEMM_COLS + 4;
    float *otile = reinterpret_cast<float *>(lds);
    float *slab = p.partial + (long)slice * p.M * p.n_total;
    const int o_row = tid >> 5;                 // 0..15
    const int o_col = (tid & 31) * 8;           // 8 consecutive columns
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        if (t < tiles) {
            __syncthreads();
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int r = 0; r < 4; ++r) otile[(4 * g + r) * OP + 128 * blk + 64 * h + 4 * c + (wave & 3)] = acc[h][t][r];
            __syncthreads();
            const int m = m0 + 16 * t + o_row;
            const int n_seg = col0 + o_col;
            if (m < p.M && n_seg < seg.N) {
                const f4 v0 = *reinterpret_cast<const f4 *>(otile + o_row * OP + o_col);
                const f4 v1 = *reinterpret_cast<const f4 *>(otile + o_row * OP + o_col + 4);
                const int n = seg.col0 + n_seg;
                if (p.direct) {
                    h8 o;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        o[e] = matmul_epilogue(p, v0[e], m, n + e);
                        o[4 + e] = matmul_epilogue(p, v1[e], m, n + 4 + e);
                    }
                    *reinterpret_cast<h8 *>(p.c + (long)m * p.ldc + n) = o;
                } else {
                    float *dst = slab + (long)m * p.n_total + n;
                    *reinterpret_cast<f4 *>(dst) = v0;
                    *reinterpret_cast<f4 *>(dst + 4) = v1;
                }
            }
        }
    }
}

void gemm_fill_plan(MatmulParams &p) {
    int unit0 = 0, col0 = 0;
    for (int i = 0; i < p.nseg; ++i) {
        p.seg[i].unit0 = unit0;
        p.seg[i].col0 = col0;
        unit0 += (p.seg[i].N + GEMM_COLS - 1) / GEMM_COLS;
        col0 += p.seg[i].N;
    }
    p.units = unit0;
    p.units_pad = (unit0 + 7) / 8 * 8;
    p.n_total = col0;
    p.mblocks = (p.M + GEMM_BM - 1) / GEMM_BM;
    const int steps = (p.K + 31) / 32;
    const long tiles = (long)p.units * p.mblocks;
    // one round of workgroups (2 per CU); fewer slices for bigger M, whose slabs are bigger (at M = 100 up to
    // 16 slices: matrices with few column units need them to fill the GPU, and the slab traffic costs less
    // than idle compute units)
    static const int capacity = env_int("SMH_GEMM_WGS", 512);
    int ks = (int)(capacity / tiles);
    static const int cap_num = env_int("SMH_GEMM_KSCAP", 1600);
    int cap = cap_num / (p.M > 0 ? p.M : 1);
    if (cap > SMH_MAX_KSPLIT) cap = SMH_MAX_KSPLIT;
    if (ks > cap) ks = cap;
    if (ks > steps / GEMM_STAGES) ks = steps / GEMM_STAGES;
    if (ks < 1) ks = 1;
    p.steps_per_slice = (steps + ks - 1) / ks;
    p.ksplit = (steps + p.steps_per_slice - 1) / p.steps_per_slice;
}

int gemm_launch(const MatmulParams &p, hipStream_t stream) {
    dim3 grid((unsigned)((long)p.units_pad * p.mblocks * p.ksplit));
    hipLaunchKernelGGL(q40_gemm_kernel, grid, dim3(GEMM_THREADS), GEMM_LDS, stream, p);
    return launch_status();
}

}  // namespace smh
