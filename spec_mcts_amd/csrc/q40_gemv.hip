// Q4_0 dequant + matmul for small batches (M <= 16): c[M,N] = a[M,K] . deq(W)[K,N].
//
// The weight is streamed exactly once, in its checkpoint layout (bytes [K, N/2], scales
// [K, N/64]); the kernel is bound by HBM bandwidth.  Algorithmic traffic per launch:
// N*K/2 + 2*N*K/64 + 2*M*K + 2*M*N bytes.
//
// Work decomposition
//   * a workgroup owns one 128-column block (one 64-byte row of packed nibbles per k) and a slice
//     of K; its 4 waves take alternate 32-row steps of that slice;
//   * inside a step, lane l = 16*g + c loads the dword at byte 4c of rows k0 + 8g .. k0 + 8g + 7,
//     i.e. 8 k-values of 8 columns.  Byte-permutes pair the same nibble of two consecutive rows,
//     one AND-OR drops the pair into the mantissa of fp16 1024.0, one packed fp16 op recovers the
//     exact integer code and one packed multiply applies the per-row scales -> the fp16 value the
//     reference dequantiser produces, already in the register layout of the B operand of
//     v_mfma_f32_16x16x32_f16 (lane = column, 8 consecutive k per lane).  The reduction over the
//     lanes' k-groups happens inside the matrix core; rows of A are the (up to 16) batch rows.
//   * partial sums of the waves are added through LDS; partial sums of the K-slices are handed to
//     the last workgroup to arrive (device-scope counter), which adds them in a fixed order, so
//     results do not depend on scheduling.  The counter is left at zero for the next launch.
//
// blockIdx.x = slice * nb_pad + block with nb_pad a multiple of 8: workgroups are dealt round-robin
// to the 8 XCDs, so all K-slices of a column block run behind the same L2.
#include "smh_common.hpp"

namespace smh {

constexpr int GEMV_WAVES = 4;
constexpr int GEMV_THREADS = GEMV_WAVES * WAVE;
constexpr int GEMV_COUNTER_SLOTS = 4096;   // uint32 counters at the start of the workspace

struct GemvParams {
    const half_t *a;
    const uint8_t *w;
    const half_t *s;
    half_t *c;
    const half_t *resid;
    float *partial;          // [ksplit][M][N]
    uint32_t *counters;      // [nb]
    long lda, ldc, ldr;
    int M, K, N;
    int nb, nb_pad;          // column blocks (N/128), padded to a multiple of 8
    int ksplit;              // K slices
    int steps_per_slice;     // 32-row steps per slice (multiple of GEMV_WAVES)
    int epilogue;
};

__device__ __forceinline__ half_t gemv_epilogue(const GemvParams &p, float acc, int m, int n) {
    half_t v = (half_t)acc;
    if (p.epilogue == SMH_EPI_RESIDUAL) v = (half_t)((float)p.resid[(long)m * p.ldr + n] + (float)v);
    return v;
}

__global__ __launch_bounds__(GEMV_THREADS) void q40_gemv_kernel(GemvParams p) {
    __shared__ float red[GEMV_WAVES][16][128];
    __shared__ uint32_t s_last;

    const int block = blockIdx.x % p.nb_pad;
    const int slice = blockIdx.x / p.nb_pad;
    if (block >= p.nb) return;
    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int c = lane & 15;
    const int g = lane >> 4;

    const long w_row = p.N / 2;            // bytes per k
    const long s_row = p.N / 64;           // scales per k
    const uint8_t *wp = p.w + (long)block * 64 + 4 * c;
    const half_t *sp = p.s + (long)block * 2;
    const int m_a = min(c, p.M - 1);       // row of A this lane feeds (rows >= M are never stored)
    const half_t *ap = p.a + (long)m_a * p.lda;

    f4 acc[2][4];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int b = 0; b < 4; ++b) acc[h][b] = f4{0.f, 0.f, 0.f, 0.f};

    const int step0 = slice * p.steps_per_slice;
    const int step1 = min(step0 + p.steps_per_slice, (p.K + 31) / 32);
    for (int step = step0 + wave; step < step1; step += GEMV_WAVES) {
        const int k0 = step * 32 + 8 * g;
        // ---- loads: 8 weight dwords, 8 scale pairs, 8 activations ----
        uint32_t wv[8], sv[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int k = min(k0 + i, p.K - 1);
            wv[i] = *reinterpret_cast<const uint32_t *>(wp + (long)k * w_row);
            sv[i] = *reinterpret_cast<const uint32_t *>(sp + (long)k * s_row);
        }
        h8 av;
        if (k0 < p.K) {
            av = *reinterpret_cast<const h8 *>(ap + k0);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) av[i] = (half_t)0.f;
        }
        // ---- decode ----
#pragma unroll
        for (int i = 0; i < 8; ++i) wv[i] ^= NIBBLE_FLIP;
        h2 s_hi[4], s_lo[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            s_hi[j] = as_h2(pack_lo16(sv[2 * j], sv[2 * j + 1]));   // scales of columns 0..63
            s_lo[j] = as_h2(pack_hi16(sv[2 * j], sv[2 * j + 1]));   // scales of columns 64..127
        }
#define SMH_GEMV_BYTE(B)                                                            \
        {                                                                           \
            h2 bh[4], bl[4];                                                        \
            _Pragma("unroll") for (int j = 0; j < 4; ++j) {                         \
                uint32_t pr = pair_bytes<B>(wv[2 * j], wv[2 * j + 1]);              \
                bh[j] = codes_high(pr) * s_hi[j];                                   \
                bl[j] = codes_low(pr) * s_lo[j];                                    \
            }                                                                       \
            h8 vb_h = {bh[0].x, bh[0].y, bh[1].x, bh[1].y, bh[2].x, bh[2].y, bh[3].x, bh[3].y}; \
            h8 vb_l = {bl[0].x, bl[0].y, bl[1].x, bl[1].y, bl[2].x, bl[2].y, bl[3].x, bl[3].y}; \
            acc[0][B] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, vb_h, acc[0][B], 0, 0, 0);   \
            acc[1][B] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, vb_l, acc[1][B], 0, 0, 0);   \
        }
        SMH_GEMV_BYTE(0)
        SMH_GEMV_BYTE(1)
        SMH_GEMV_BYTE(2)
        SMH_GEMV_BYTE(3)
#undef SMH_GEMV_BYTE
    }

    // ---- add the 4 waves' partial sums through LDS ----
    // accumulator element r of lane (g, c) is row m = 4g + r, column 64h + 4c + b of the block
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = 4 * g + r;
                if (m < p.M) red[wave][m][64 * h + 4 * c + b] = acc[h][b][r];
            }
    __syncthreads();

    const int n_local = tid & 127;
    const int n = block * 128 + n_local;
    const int m_first = tid >> 7;           // 0 or 1; rows m_first, m_first + 2, ...
    float sum[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int m = m_first + 2 * j;
        sum[j] = 0.f;
        if (m < p.M) {
#pragma unroll
            for (int wv_ = 0; wv_ < GEMV_WAVES; ++wv_) sum[j] += red[wv_][m][n_local];
        }
    }

    if (p.ksplit == 1) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int m = m_first + 2 * j;
            if (m < p.M) p.c[(long)m * p.ldc + n] = gemv_epilogue(p, sum[j], m, n);
        }
        return;
    }

    // ---- hand the slice's sums to the last workgroup of this column block ----
    const long slice_stride = (long)p.M * p.N;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int m = m_first + 2 * j;
        if (m < p.M) store_coherent(p.partial + slice * slice_stride + (long)m * p.N + n, sum[j]);
    }
    __threadfence();
    __syncthreads();
    if (tid == 0) {
        uint32_t prev = __hip_atomic_fetch_add(p.counters + block, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        s_last = (prev == (uint32_t)p.ksplit - 1u) ? 1u : 0u;
    }
    __syncthreads();
    if (!s_last) return;
    __threadfence();
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int m = m_first + 2 * j;
        if (m < p.M) {
            float tot = 0.f;
            for (int sl = 0; sl < p.ksplit; ++sl)
                tot += load_coherent(p.partial + sl * slice_stride + (long)m * p.N + n);
            p.c[(long)m * p.ldc + n] = gemv_epilogue(p, tot, m, n);
        }
    }
    if (tid == 0) __hip_atomic_store(p.counters + block, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Slices are chosen so that about 4 workgroups per CU are in flight (256 CUs) while every wave still
// has at least one step to do.
static void gemv_plan(int N, int K, int *ksplit, int *steps_per_slice) {
    const int nb = N / 128;
    const int steps = (K + 31) / 32;
    int want = (1024 + nb - 1) / nb;
    int max_split = (steps + GEMV_WAVES - 1) / GEMV_WAVES;
    int ks = want < 1 ? 1 : want;
    if (ks > max_split) ks = max_split;
    int sps = (steps + ks - 1) / ks;
    sps = (sps + GEMV_WAVES - 1) / GEMV_WAVES * GEMV_WAVES;
    ks = (steps + sps - 1) / sps;
    *ksplit = ks;
    *steps_per_slice = sps;
}

}  // namespace smh

extern "C" size_t smh_q40_matmul_workspace_bytes(int max_m, int max_n) {
    // counters + K-slice partial sums.
    // GEMV (M <= 16): ksplit * N never exceeds max(N, 1024 column blocks * 128 columns).
    // GEMM (M > 16) : ksplit * M * N never exceeds 512 tiles of 128 x 128 when K is split at all.
    size_t m = (size_t)(max_m < 1 ? 1 : (max_m > SMH_GEMV_MAX_M ? SMH_GEMV_MAX_M : max_m));
    size_t floats = ((size_t)(max_n > 131072 ? max_n : 131072) + 128) * m;
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
    GemvParams p;
    p.a = (const half_t *)a; p.w = (const uint8_t *)b_w; p.s = (const half_t *)b_s;
    p.c = (half_t *)c; p.resid = (const half_t *)residual;
    p.lda = lda; p.ldc = ldc; p.ldr = ldr;
    p.M = M; p.K = K; p.N = N;
    p.nb = N / 128;
    p.nb_pad = (p.nb + 7) / 8 * 8;
    p.epilogue = epilogue;
    gemv_plan(N, K, &p.ksplit, &p.steps_per_slice);
    SMH_REQUIRE(p.nb <= GEMV_COUNTER_SLOTS, "smh_q40_gemv: N=%d too large (max %d)", N, GEMV_COUNTER_SLOTS * 128);
    p.counters = (uint32_t *)workspace;
    p.partial = (float *)((char *)workspace + (size_t)GEMV_COUNTER_SLOTS * 4);
    if (p.ksplit > 1) {
        size_t need = (size_t)GEMV_COUNTER_SLOTS * 4 + (size_t)p.ksplit * M * N * sizeof(float);
        SMH_REQUIRE(workspace && workspace_bytes >= need, "smh_q40_gemv: workspace %zu < %zu bytes", workspace_bytes, need);
    }
    dim3 grid((unsigned)(p.nb_pad * p.ksplit));
    hipLaunchKernelGGL(q40_gemv_kernel, grid, dim3(GEMV_THREADS), 0, (hipStream_t)stream, p);
    return launch_status();
}
