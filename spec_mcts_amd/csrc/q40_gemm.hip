// Q4_0 dequant + matmul for large batches (decode at B = 100, prefill): c[M,N] = a[M,K] . deq(W)[K,N].
//
// A workgroup owns 128 rows of A, one 128-column block of the weight (one 64-byte packed row per
// k) and a slice of K.  Per 32-row step
//   * the 128 x 32 tile of A is staged in LDS (row pitch 40 halves, so the 16 rows read by one
//     ds_read_b128 wavefront pass fall on distinct banks);
//   * every wave loads the step's 8 weight dwords per lane, but decodes only ONE byte position
//     (wave w <-> byte w of each dword): 32 of the block's 128 columns.  Decoding is the same
//     perm / and-or / packed-fp16 sequence as the GEMV and lands directly in the B-operand layout
//     of v_mfma_f32_16x16x32_f16, so dequantised weights never travel through LDS or HBM;
//   * the wave multiplies its two B operands with all (up to 8) 16-row tiles of A.
// K-slices are combined as in the GEMV: coherent partial sums, last workgroup adds in fixed order.
//
// At M = 100 the work sits on the ridge of the roofline: 2*M*N*K flops against
// N*K*0.53125 + 2*M*(K+N) bytes.
#include "smh_common.hpp"

namespace smh {

constexpr int GEMM_BM = 128;
constexpr int GEMM_THREADS = 256;
constexpr int GEMM_PITCH = 40;             // halves per LDS row of the A tile
constexpr int GEMM_COUNTER_SLOTS = 4096;

struct GemmParams {
    const half_t *a;
    const uint8_t *w;
    const half_t *s;
    half_t *c;
    const half_t *resid;
    float *partial;
    uint32_t *counters;
    long lda, ldc, ldr;
    int M, K, N;
    int nb, mblocks, ksplit, steps_per_slice, epilogue;
};

__global__ __launch_bounds__(GEMM_THREADS) void q40_gemm_kernel(GemmParams p) {
    __shared__ __attribute__((aligned(16))) half_t a_tile[GEMM_BM][GEMM_PITCH];
    __shared__ uint32_t s_last;

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int c = lane & 15;
    const int g = lane >> 4;
    int bid = blockIdx.x;
    const int block = bid % p.nb;  bid /= p.nb;
    const int mb = bid % p.mblocks;
    const int slice = bid / p.mblocks;
    const int m0 = mb * GEMM_BM;
    const int m_count = min(GEMM_BM, p.M - m0);
    const int tiles = (m_count + 15) / 16;

    const long w_row = p.N / 2;
    const long s_row = p.N / 64;
    const uint8_t *wp = p.w + (long)block * 64 + 4 * c;
    const half_t *sp = p.s + (long)block * 2;
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
    for (int step = step0; step < step1; ++step) {
        const int kb = step * 32;
        // ---- global loads for this step ----
        u32x4 sa0 = {0, 0, 0, 0}, sa1 = {0, 0, 0, 0};
        if (kb + st_col < p.K) sa0 = *reinterpret_cast<const u32x4 *>(st_src + kb);
        if (kb + st_col + 8 < p.K) sa1 = *reinterpret_cast<const u32x4 *>(st_src + kb + 8);
        const int k0 = kb + 8 * g;
        uint32_t wv[8], sv[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int k = min(k0 + i, p.K - 1);
            wv[i] = *reinterpret_cast<const uint32_t *>(wp + (long)k * w_row) ^ NIBBLE_FLIP;
            sv[i] = *reinterpret_cast<const uint32_t *>(sp + (long)k * s_row);
        }
        __syncthreads();                    // previous step's reads of a_tile are done
        *reinterpret_cast<u32x4 *>(&a_tile[st_row][st_col]) = sa0;
        *reinterpret_cast<u32x4 *>(&a_tile[st_row][st_col + 8]) = sa1;
        // ---- decode this wave's byte position ----
        h2 bh[4], bl[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint32_t pr = __builtin_amdgcn_perm(wv[2 * j + 1], wv[2 * j], sel);
            bh[j] = codes_high(pr) * as_h2(pack_lo16(sv[2 * j], sv[2 * j + 1]));
            bl[j] = codes_low(pr) * as_h2(pack_hi16(sv[2 * j], sv[2 * j + 1]));
        }
        h8 vb_h = {bh[0].x, bh[0].y, bh[1].x, bh[1].y, bh[2].x, bh[2].y, bh[3].x, bh[3].y};
        h8 vb_l = {bl[0].x, bl[0].y, bl[1].x, bl[1].y, bl[2].x, bl[2].y, bl[3].x, bl[3].y};
        __syncthreads();                    // a_tile holds this step
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            if (t < tiles) {
                h8 av = *reinterpret_cast<const h8 *>(&a_tile[t * 16 + c][8 * g]);
                acc[0][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, vb_h, acc[0][t], 0, 0, 0);
                acc[1][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, vb_l, acc[1][t], 0, 0, 0);
            }
        }
    }

    // accumulator element r of acc[h][t] is row m0 + 16t + 4g + r, column 128*block + 64h + 4c + wave
    const int n_base = block * 128 + 4 * c + wave;
    if (p.ksplit == 1) {
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int t = 0; t < 8; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int m = m0 + 16 * t + 4 * g + r;
                    const int n = n_base + 64 * h;
                    if (m < p.M) {
                        half_t v = (half_t)acc[h][t][r];
                        if (p.epilogue == SMH_EPI_RESIDUAL)
                            v = (half_t)((float)p.resid[(long)m * p.ldr + n] + (float)v);
                        p.c[(long)m * p.ldc + n] = v;
                    }
                }
        return;
    }

    const long slice_stride = (long)p.M * p.N;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int t = 0; t < 8; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = m0 + 16 * t + 4 * g + r;
                if (m < p.M)
                    store_coherent(p.partial + slice * slice_stride + (long)m * p.N + n_base + 64 * h, acc[h][t][r]);
            }
    uint32_t *counter = p.counters + mb * p.nb + block;
    if (!arrive_is_last(counter, (uint32_t)p.ksplit, &s_last)) return;
    // the last workgroup adds the slices in order; thread t handles column t%128, rows t/128, +2, ...
    const int n = block * 128 + (tid & 127);
    for (int mm = tid >> 7; mm < m_count; mm += 2) {
        const int m = m0 + mm;
        float tot = 0.f;
        for (int sl = 0; sl < p.ksplit; ++sl)
            tot += load_coherent(p.partial + sl * slice_stride + (long)m * p.N + n);
        half_t v = (half_t)tot;
        if (p.epilogue == SMH_EPI_RESIDUAL) v = (half_t)((float)p.resid[(long)m * p.ldr + n] + (float)v);
        p.c[(long)m * p.ldc + n] = v;
    }
    arrive_reset(counter);
}

}  // namespace smh

extern "C" int smh_q40_gemm(const void *a, int M, int K, long lda, const void *b_w, const void *b_s, int N,
                            void *c, long ldc, int epilogue, const void *residual, long ldr,
                            void *workspace, size_t workspace_bytes, smh_stream_t stream) {
    using namespace smh;
    SMH_REQUIRE(M >= 0, "smh_q40_gemm: M=%d", M);
    SMH_REQUIRE(N > 0 && N % 128 == 0, "smh_q40_gemm: N=%d must be a positive multiple of 128", N);
    SMH_REQUIRE(K > 0 && K % 8 == 0, "smh_q40_gemm: K=%d must be a positive multiple of 8", K);
    SMH_REQUIRE(lda >= K && ldc >= N, "smh_q40_gemm: lda=%ld ldc=%ld too small", lda, ldc);
    SMH_REQUIRE(lda % 8 == 0, "smh_q40_gemm: lda=%ld must be a multiple of 8 (128-bit loads)", lda);
    SMH_REQUIRE(epilogue == SMH_EPI_NONE || epilogue == SMH_EPI_RESIDUAL, "smh_q40_gemm: epilogue=%d", epilogue);
    if (M == 0) return 0;
    SMH_REQUIRE(a && b_w && b_s && c, "smh_q40_gemm: null pointer");
    SMH_REQUIRE(epilogue != SMH_EPI_RESIDUAL || (residual && ldr >= N), "smh_q40_gemm: residual missing");
    GemmParams p;
    p.a = (const half_t *)a; p.w = (const uint8_t *)b_w; p.s = (const half_t *)b_s;
    p.c = (half_t *)c; p.resid = (const half_t *)residual;
    p.lda = lda; p.ldc = ldc; p.ldr = ldr;
    p.M = M; p.K = K; p.N = N; p.epilogue = epilogue;
    p.nb = N / 128;
    p.mblocks = (M + GEMM_BM - 1) / GEMM_BM;
    const int steps = (K + 31) / 32;
    const long tiles = (long)p.nb * p.mblocks;
    int ks = (int)(512 / tiles);
    if (ks < 1) ks = 1;
    if (ks > steps / 4) ks = steps / 4 > 0 ? steps / 4 : 1;
    if (tiles > GEMM_COUNTER_SLOTS) ks = 1;
    p.steps_per_slice = (steps + ks - 1) / ks;
    p.ksplit = (steps + p.steps_per_slice - 1) / p.steps_per_slice;
    p.counters = (uint32_t *)workspace;
    p.partial = (float *)((char *)workspace + (size_t)GEMM_COUNTER_SLOTS * 4);
    if (p.ksplit > 1) {
        size_t need = (size_t)GEMM_COUNTER_SLOTS * 4 + (size_t)p.ksplit * M * N * sizeof(float);
        SMH_REQUIRE(workspace && workspace_bytes >= need, "smh_q40_gemm: workspace %zu < %zu bytes", workspace_bytes, need);
    }
    dim3 grid((unsigned)(tiles * p.ksplit));
    hipLaunchKernelGGL(q40_gemm_kernel, grid, dim3(GEMM_THREADS), 0, (hipStream_t)stream, p);
    return launch_status();
}

extern "C" int smh_q40_matmul(const void *a, int M, int K, long lda, const void *b_w, const void *b_s, int N,
                              void *c, long ldc, int epilogue, const void *residual, long ldr,
                              void *workspace, size_t workspace_bytes, smh_stream_t stream) {
    if (M <= SMH_GEMV_MAX_M)
        return smh_q40_gemv(a, M, K, lda, b_w, b_s, N, c, ldc, epilogue, residual, ldr, workspace, workspace_bytes, stream);
    return smh_q40_gemm(a, M, K, lda, b_w, b_s, N, c, ldc, epilogue, residual, ldr, workspace, workspace_bytes, stream);
}
