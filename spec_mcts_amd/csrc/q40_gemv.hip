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
//     before decoding either, which keeps ~7 KB per wave in flight;
//   * inside a step, lane l = 16*g + c loads the 8 bytes at offset 8c of rows k0 + 8g .. k0 + 8g + 7,
//     i.e. 8 k-values of 16 columns.  Byte-permutes pair the same nibble of two consecutive rows,
//     one AND-OR drops the pair into the mantissa of fp16 1024.0, one packed fp16 op recovers the
//     exact integer code and one packed multiply applies the per-row scales -> the fp16 value the
//     reference dequantiser produces, already in the register layout of the B operand of
//     v_mfma_f32_16x16x32_f16 (lane = column, 8 consecutive k per lane).  The reduction over the
//     lanes' k-groups happens inside the matrix core; rows of A are the (up to 16) batch rows.
//   * partial sums of the waves are added through LDS; partial sums of the K-slices are handed to
//     the last workgroup to arrive (device-scope counter), which adds them in a fixed order, so
//     results do not depend on scheduling.  The counter is left at zero for the next launch.
//
// blockIdx.x = slice * pairs_pad + pair with pairs_pad a multiple of 8: workgroups are dealt
// round-robin to the 8 XCDs, so all K-slices of a column pair run behind the same L2.
#include <stdlib.h>

#include "smh_common.hpp"

namespace smh {

constexpr int GEMV_COUNTER_SLOTS = 4096;   // uint32 counters at the start of the workspace
constexpr int GEMV_MAX_SPLIT = 16;         // K slices per column pair (bounds the unrolled tail)
constexpr int GEMV_COLS = 256;             // columns per workgroup

struct GemvParams {
    const half_t *a;
    const uint8_t *w;
    const half_t *s;
    half_t *c;
    const half_t *resid;
    float *partial;          // [ksplit][M][N]
    uint32_t *counters;      // [pairs]
    long lda, ldc, ldr;
    int M, K, N;
    int pairs, pairs_pad;    // column pairs (ceil(N/256)), padded to a multiple of 8
    int ksplit;              // K slices
    int steps_per_slice;     // 32-row steps per slice (multiple of 2 * waves per workgroup)
    int epilogue;
};

__device__ __forceinline__ half_t gemv_epilogue(const GemvParams &p, float acc, int m, int n) {
    half_t v = (half_t)acc;
    if (p.epilogue == SMH_EPI_RESIDUAL) v = (half_t)((float)p.resid[(long)m * p.ldr + n] + (float)v);
    return v;
}

// registers of one 32-row step of one lane
struct GemvStep {
    u32x2 wv[8];     // 8 bytes of 8 consecutive rows
    uint32_t sv[8];  // (scale of columns 0..63, scale of columns 64..127) of this lane's block, per row
    h8 av;           // 8 activations of batch row c
};

__device__ __forceinline__ void gemv_load(GemvStep &st, const GemvParams &p, const uint8_t *wp, const half_t *sp,
                                          const half_t *ap, long w_row, long s_row, int k0) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int k = min(k0 + i, p.K - 1);
        st.wv[i] = *reinterpret_cast<const u32x2 *>(wp + (long)k * w_row);
        st.sv[i] = *reinterpret_cast<const uint32_t *>(sp + (long)k * s_row);
    }
    if (k0 < p.K) {
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
__global__ __launch_bounds__(WAVES * 64) void q40_gemv_kernel(GemvParams p) {
    extern __shared__ float red[];          // [WAVES][M][256]
    __shared__ uint32_t s_last;
    constexpr int THREADS = WAVES * 64;

    const int pair = blockIdx.x % p.pairs_pad;
    const int slice = blockIdx.x / p.pairs_pad;
    if (pair >= p.pairs) return;
    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int c = lane & 15;
    const int g = lane >> 4;

    const long w_row = p.N / 2;            // bytes per k
    const long s_row = p.N / 64;           // scales per k
    const int col0 = pair * GEMV_COLS;     // first column of this workgroup
    // lanes c >= 8 belong to the second block of the pair; when N/128 is odd the last pair has none:
    // such lanes re-read the first block (valid memory) and their results are dropped
    const bool has_block = col0 + 128 * (c >> 3) < p.N;
    const int c_ld = has_block ? c : (c & 7);
    const uint8_t *wp = p.w + (long)pair * 128 + 8 * c_ld;
    const half_t *sp = p.s + (long)pair * 4 + 2 * (c_ld >> 3);
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
        gemv_load(s0, p, wp, sp, ap, w_row, s_row, step * 32 + 8 * g);
        const bool two = step + 1 < step1;
        if (two) gemv_load(s1, p, wp, sp, ap, w_row, s_row, (step + 1) * 32 + 8 * g);
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
    const long slice_stride = (long)p.M * p.N;
    for (int idx = tid; idx < outputs; idx += THREADS) {
        float sum = 0.f;
#pragma unroll
        for (int wv_ = 0; wv_ < WAVES; ++wv_) sum += red[wv_ * outputs + idx];
        const int m = idx >> 8, n = col0 + (idx & 255);
        if (n >= p.N) continue;
        if (p.ksplit == 1) p.c[(long)m * p.ldc + n] = gemv_epilogue(p, sum, m, n);
        else store_coherent(p.partial + slice * slice_stride + (long)m * p.N + n, sum);
    }
    if (p.ksplit == 1) return;

    // ---- the last workgroup of this column pair adds the slices in a fixed order ----
    if (!arrive_is_last(p.counters + pair, (uint32_t)p.ksplit, &s_last)) return;
    for (int idx = tid; idx < outputs; idx += THREADS) {
        const int m = idx >> 8, n = col0 + (idx & 255);
        if (n >= p.N) continue;
        const float *src = p.partial + (long)m * p.N + n;
        float v[GEMV_MAX_SPLIT];
#pragma unroll
        for (int sl = 0; sl < GEMV_MAX_SPLIT; ++sl) v[sl] = (sl < p.ksplit) ? load_coherent(src + sl * slice_stride) : 0.f;
        float tot = 0.f;
#pragma unroll
        for (int sl = 0; sl < GEMV_MAX_SPLIT; ++sl) tot += v[sl];
        p.c[(long)m * p.ldc + n] = gemv_epilogue(p, tot, m, n);
    }
    arrive_reset(p.counters + pair);
}

static int env_int(const char *name, int dflt) {
    const char *v = getenv(name);
    return v ? atoi(v) : dflt;
}

// K is cut into at most GEMV_MAX_SPLIT slices so that about `target` workgroups are in flight
// (256 CUs) while every wave still has a pair of steps to do.
static void gemv_plan(int N, int K, int waves, int *ksplit, int *steps_per_slice) {
    const int pairs = (N + GEMV_COLS - 1) / GEMV_COLS;
    const int steps = (K + 31) / 32;
    static const int target_wgs = env_int("SMH_GEMV_WGS", 512);
    const int unit = 2 * waves;
    int want = (target_wgs + pairs - 1) / pairs;
    int max_split = (steps + unit - 1) / unit;
    int ks = want < 1 ? 1 : want;
    if (ks > max_split) ks = max_split;
    if (ks > GEMV_MAX_SPLIT) ks = GEMV_MAX_SPLIT;
    int sps = (steps + ks - 1) / ks;
    sps = (sps + unit - 1) / unit * unit;
    ks = (steps + sps - 1) / sps;
    *ksplit = ks;
    *steps_per_slice = sps;
}

}  // namespace smh

extern "C" size_t smh_q40_matmul_workspace_bytes(int max_m, int max_n) {
    // counters + K-slice partial sums.
    // GEMV (M <= 16): at most GEMV_MAX_SPLIT slices of [M, N] floats.
    // GEMM (M > 16) : ksplit * M * N never exceeds 512 tiles of 128 x 128 when K is split at all.
    size_t m = (size_t)(max_m < 1 ? 1 : (max_m > SMH_GEMV_MAX_M ? SMH_GEMV_MAX_M : max_m));
    size_t n = (size_t)(max_n < 128 ? 128 : max_n);
    size_t floats = n * m * smh::GEMV_MAX_SPLIT;
    if (max_m > SMH_GEMV_MAX_M && floats < (size_t)512 * 128 * 128) floats = (size_t)512 * 128 * 128;
    return (size_t)smh::GEMV_COUNTER_SLOTS * 4 + floats * sizeof(float);
}

extern "C" int smh_q40_gemv(const void *a, int M, int K, long lda, const void *b_w, const void *b_s, int N,
                            void *c, long ldc, int epilogue, const void *residual, long ldr,
                            void *workspace, size_t workspace_bytes, smh_stream_t stream) {
    using namespace smh;
    SMH_REQUIRE(M >= 0 && M <= SMH_GEMV_MAX_M, "smh_q40_gemv: M=%d outside [0,%d]", M, SMH_GEMV_MAX_M);
    SMH_REQUIRE(N > 0 && N % 128 == 0, "smh_q40_gemv: N=%d must be a positive multiple of 128", N);
    SMH_REQUIRE(K > 0 && K % 8 == 0, "smh_q40_gemv: K=%d must be a positive multiple of 8", K);
    SMH_REQUIRE(lda >= K && ldc >= N, "smh_q40_gemv: lda=%ld ldc=%ld too small", lda, ldc);
    SMH_REQUIRE(lda % 8 == 0, "smh_q40_gemv: lda=%ld must be a multiple of 8 (128-bit loads)", lda);
    SMH_REQUIRE(epilogue == SMH_EPI_NONE || epilogue == SMH_EPI_RESIDUAL, "smh_q40_gemv: epilogue=%d", epilogue);
    if (M == 0) return 0;
    SMH_REQUIRE(a && b_w && b_s && c, "smh_q40_gemv: null pointer");
    SMH_REQUIRE(epilogue != SMH_EPI_RESIDUAL || (residual && ldr >= N), "smh_q40_gemv: residual missing");
    static const int waves_pref = env_int("SMH_GEMV_WAVES", 4);
    int waves = waves_pref;
    while (waves > 2 && (size_t)waves * M * GEMV_COLS * sizeof(float) > 48 * 1024) waves >>= 1;   // LDS budget
    GemvParams p;
    p.a = (const half_t *)a; p.w = (const uint8_t *)b_w; p.s = (const half_t *)b_s;
    p.c = (half_t *)c; p.resid = (const half_t *)residual;
    p.lda = lda; p.ldc = ldc; p.ldr = ldr;
    p.M = M; p.K = K; p.N = N;
    p.pairs = (N + GEMV_COLS - 1) / GEMV_COLS;
    p.pairs_pad = (p.pairs + 7) / 8 * 8;
    p.epilogue = epilogue;
    gemv_plan(N, K, waves, &p.ksplit, &p.steps_per_slice);
    SMH_REQUIRE(p.pairs <= GEMV_COUNTER_SLOTS, "smh_q40_gemv: N=%d too large (max %d)", N, GEMV_COUNTER_SLOTS * GEMV_COLS);
    p.counters = (uint32_t *)workspace;
    p.partial = (float *)((char *)workspace + (size_t)GEMV_COUNTER_SLOTS * 4);
    if (p.ksplit > 1) {
        size_t need = (size_t)GEMV_COUNTER_SLOTS * 4 + (size_t)p.ksplit * M * N * sizeof(float);
        SMH_REQUIRE(workspace && workspace_bytes >= need, "smh_q40_gemv: workspace %zu < %zu bytes", workspace_bytes, need);
    }
    dim3 grid((unsigned)(p.pairs_pad * p.ksplit));
    size_t lds = (size_t)waves * M * GEMV_COLS * sizeof(float);
    if (waves == 2) hipLaunchKernelGGL(q40_gemv_kernel<2>, grid, dim3(128), lds, (hipStream_t)stream, p);
    else if (waves == 8) hipLaunchKernelGGL(q40_gemv_kernel<8>, grid, dim3(512), lds, (hipStream_t)stream, p);
    else hipLaunchKernelGGL(q40_gemv_kernel<4>, grid, dim3(256), lds, (hipStream_t)stream, p);
    return launch_status();
}
