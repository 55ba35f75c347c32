// fp16 linear without bias for the vocabulary projection (lm_head) and the token embedding gather.
//
//   out[M, N] = x[M, K] . W[N, K]^T      fp16 operands, fp32 accumulation, one rounding to fp16
//
// W is the checkpoint tensor of nn.Linear (row n = the K weights of output n, contiguous), read exactly once per
// 128-row block of x; at the 7B architecture it is 262 MB, the largest tensor of a decode step, so the kernel is bound by
// HBM bandwidth: algorithmic bytes N*K*2 + M*K*2 + M*N*2.
//
// A workgroup of 4 waves owns 128 outputs (rows of W) and up to 128 rows of x and walks K in stages of 64 values (one
// 128-byte line per row).  Everything a stage needs goes global -> LDS by DMA (global_load_lds) into a ring:
//   * wave w moves and consumes the 32 rows of W it owns (4 DMA instructions of 8 rows x 128 B): that part of the ring is
//     private to the wave;
//   * the x tile (16 rows per tile, up to 8 tiles) is shared by the workgroup, its DMA instructions dealt evenly to the
//     waves so that one vmcnt constant serves all; one bare s_barrier per stage publishes it and frees the oldest slot.
// Inside a 128-byte row the 16-byte chunks are stored XOR-swizzled (chunk q of row r sits in slot q ^ ((r >> 1) & 7)): the
// 16 lanes that read the same chunk of 16 different rows then cover all 64 LDS banks exactly once (ds_read_b128 without
// conflicts), while the global side still reads whole lines.
// The rows of W are the A operand of v_mfma_f32_16x16x32_f16 and the rows of x the B operand, so a lane ends up with four
// consecutive outputs n of one row m and stores them as 8 bytes.
#include "smh_common.hpp"

namespace smh {

constexpr int HEAD_BN = 128;                   // outputs (rows of W) per workgroup
constexpr int HEAD_BM = 128;                   // rows of x per workgroup
constexpr int HEAD_WAVES = 4;
constexpr int HEAD_KS = 64;                    // K values per stage (128 bytes per row)
constexpr int HEAD_W_BYTES = HEAD_BN * 128;    // 16 KB per stage
constexpr int HEAD_LDS_MAX = 160 * 1024;
// ring slots for TILES 16-row tiles of x: four (six and eight, where the compute unit's LDS holds them, measured 2-3 % slower:
// the kernel does not wait on memory latency)
constexpr int HEAD_MAX_STAGES = 4;
constexpr int head_stages(int tiles) {
    const int fit = HEAD_LDS_MAX / (HEAD_W_BYTES + tiles * 16 * 128);
    return fit > HEAD_MAX_STAGES ? HEAD_MAX_STAGES : fit;
}

typedef const __attribute__((address_space(1))) void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;

struct HeadParams {
    const half_t *x;
    const half_t *w;
    half_t *out;
    long ldx, ldo;
    int M, N, K;
    int vec_store;           // out and ldo allow 8-byte stores of four outputs
};

template <int N_>
__device__ __forceinline__ void head_wait_dma() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N_) : "memory"); }
// at most `left` (0 .. MAX) stages of PER instructions may stay in flight
template <int PER, int MAX>
__device__ __forceinline__ void head_wait_stages(int left) {
    if constexpr (MAX == 0) head_wait_dma<0>();
    else {
        if (left >= MAX) head_wait_dma<MAX * PER>();
        else head_wait_stages<PER, MAX - 1>(left);
    }
}

// TILES: 16-row tiles of x a workgroup multiplies (1..8); XD = DMA instructions of the x tile per wave and stage
template <int TILES>
__global__ __launch_bounds__(HEAD_WAVES * 64) void f16_head_kernel(HeadParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr int X_BYTES = TILES * 16 * 128;
    constexpr int STAGE = HEAD_W_BYTES + X_BYTES;
    constexpr int XD = (2 * TILES + HEAD_WAVES - 1) / HEAD_WAVES;
    constexpr int PER = 4 + XD;                       // DMA instructions per wave and stage
    constexpr int HEAD_STAGES = head_stages(TILES);
    static_assert(HEAD_STAGES >= 3 && (HEAD_STAGES - 2) * PER <= 63, "vmcnt is a 6-bit counter");

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int c = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * HEAD_BN;
    const int m0 = blockIdx.y * HEAD_BM;

    // ---- DMA addressing: lane l of an instruction moves slot q = l % 8 of row r = l / 8 of an 8-row group ----
    const int d_r = lane >> 3, d_q = lane & 7;
    // W: this wave's rows 32 w + 8 i + d_r (i = 0..3); rows past N repeat row N - 1 (their outputs are not stored)
    uint32_t w_off[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int rr = 32 * wave + 8 * i + d_r;                          // row inside the workgroup's 128
        const int row = min(n0 + rr, p.N - 1);
        w_off[i] = (uint32_t)(((long)(row - n0) * p.K + 8 * (d_q ^ ((rr >> 1) & 7))) * 2);     // bytes from row n0, column 0 (may be negative only if N <= n0: excluded by the grid)
    }
    const uint8_t *w_base = reinterpret_cast<const uint8_t *>(p.w + (long)n0 * p.K);
    // x: 8-row groups 0 .. 2 TILES - 1 dealt to the waves; a wave without a group left repeats the last one
    uint32_t x_off[XD];
    int x_grp[XD];
#pragma unroll
    for (int j = 0; j < XD; ++j) {
        const int grp = min(wave + HEAD_WAVES * j, 2 * TILES - 1);
        const int rr = 8 * grp + d_r;
        const int row = min(m0 + rr, p.M - 1);
        x_grp[j] = grp;
        x_off[j] = (uint32_t)(((long)row * p.ldx + 8 * (d_q ^ ((rr >> 1) & 7))) * 2);
    }
    const uint8_t *x_base = reinterpret_cast<const uint8_t *>(p.x);

    // Workgroup j starts at stage j of K and wraps.  The rows of W are K * 2 bytes apart (8 KB at the 7B shape), so with every
    // workgroup on the same stage all 128 x 251 row pieces in flight have the same low address bits and fall on a few memory
    // channels: 59.6 us per launch at the 7B shape; staggered, 47.8 us (5.5 TB/s).  The order of the fp32 additions of an output
    // then depends on its block of 128 outputs, not on anything that varies between runs.
    const int n_stages = p.K / HEAD_KS;
    const int rot = (int)(blockIdx.x % (unsigned)n_stages);
    auto issue = [&](int stage_i, int slot) {
        uint8_t *st = lds + slot * STAGE;
        int stage_k = stage_i + rot;
        if (stage_k >= n_stages) stage_k -= n_stages;
        const long kb = (long)stage_k * HEAD_KS * 2;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            __builtin_amdgcn_global_load_lds((gptr_t)(w_base + kb + w_off[i]), (lptr_t)(st + (32 * wave + 8 * i) * 128), 16, 0, 0);
#pragma unroll
        for (int j = 0; j < XD; ++j)
            __builtin_amdgcn_global_load_lds((gptr_t)(x_base + kb + x_off[j]), (lptr_t)(st + HEAD_W_BYTES + x_grp[j] * 1024), 16, 0, 0);
    };

    f4 acc[2][TILES];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int t = 0; t < TILES; ++t) acc[a][t] = f4{0.f, 0.f, 0.f, 0.f};

#pragma unroll
    for (int i = 0; i < HEAD_STAGES - 1; ++i)
        if (i < n_stages) issue(i, i);

    // operand reads: row (16 a + c of the wave's 32 | 16 t + c of the x tile), logical chunk 4 j + g of the stage
    auto compute = [&](const uint8_t *st) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            h8 wa[2], xb[TILES];
#pragma unroll
            for (int a = 0; a < 2; ++a) {
                const int rr = 32 * wave + 16 * a + c;
                wa[a] = *reinterpret_cast<const h8 *>(st + rr * 128 + (((4 * j + g) ^ ((rr >> 1) & 7)) << 4));
            }
#pragma unroll
            for (int t = 0; t < TILES; ++t) {
                const int rr = 16 * t + c;
                xb[t] = *reinterpret_cast<const h8 *>(st + HEAD_W_BYTES + rr * 128 + (((4 * j + g) ^ ((rr >> 1) & 7)) << 4));
            }
#pragma unroll
            for (int t = 0; t < TILES; ++t)
#pragma unroll
                for (int a = 0; a < 2; ++a) acc[a][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wa[a], xb[t], acc[a][t], 0, 0, 0);
        }
    };

    int slot = 0;
    int i = 0;
    // main part: a refill per iteration, so exactly HEAD_STAGES - 1 stages are in flight when the wait is reached
#pragma unroll 1
    for (; i + HEAD_STAGES - 1 < n_stages; ++i) {
        head_wait_dma<(HEAD_STAGES - 2) * PER>();                         // stage i of this wave has landed ...
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); // ... and everyone's; everyone is done with stage i - 1
        issue(i + HEAD_STAGES - 1, slot == 0 ? HEAD_STAGES - 1 : slot - 1);
        compute(lds + slot * STAGE);
        slot = slot == HEAD_STAGES - 1 ? 0 : slot + 1;
    }
    // drain: no refills; `left` younger stages are still in flight
#pragma unroll 1
    for (; i < n_stages; ++i) {
        head_wait_stages<PER, HEAD_STAGES - 2>(n_stages - 1 - i);
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        compute(lds + slot * STAGE);
        slot = slot == HEAD_STAGES - 1 ? 0 : slot + 1;
    }

    // element r of acc[a][t] in lane (g, c): output n = n0 + 32 w + 16 a + 4 g + r of row m = m0 + 16 t + c
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
        const int m = m0 + 16 * t + c;
        if (m >= p.M) continue;
#pragma unroll
        for (int a = 0; a < 2; ++a) {
            const int n = n0 + 32 * wave + 16 * a + 4 * g;
            half_t *dst = p.out + (long)m * p.ldo + n;
            if (n + 3 < p.N && p.vec_store) {
                *reinterpret_cast<h4 *>(dst) = h4{(half_t)acc[a][t][0], (half_t)acc[a][t][1], (half_t)acc[a][t][2], (half_t)acc[a][t][3]};
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (n + r < p.N) dst[r] = (half_t)acc[a][t][r];
            }
        }
    }
}

// ---- embedding gather: out[m][:] = table[tokens[m]][:] ------------------------------------------------------------
__global__ __launch_bounds__(256) void embedding_kernel(const int64_t *__restrict__ tokens, const half_t *__restrict__ table,
                                                        half_t *__restrict__ out, int dim, int vocab) {
    const int m = blockIdx.x;
    long tok = tokens[m];
    tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);              // an id outside the table reads its nearest row, never past it
    const u32x4 *src = reinterpret_cast<const u32x4 *>(table + tok * dim);
    u32x4 *dst = reinterpret_cast<u32x4 *>(out + (long)m * dim);
    for (int i = threadIdx.x; i < dim / 8; i += 256) dst[i] = src[i];
}

typedef void (*head_kernel_t)(HeadParams);

}  // namespace smh

using namespace smh;

extern "C" int smh_f16_linear(const void *x, int M, int K, long ldx, const void *w, int N, void *out, long ldo, smh_stream_t stream) {
    const char *who = "smh_f16_linear";
    SMH_REQUIRE(M >= 0 && N > 0 && K > 0 && K % HEAD_KS == 0, "%s: M=%d N=%d K=%d (K must be a positive multiple of %d)", who, M, N, K, HEAD_KS);
    SMH_REQUIRE(ldx >= K && ldx % 8 == 0 && ldo >= N, "%s: ldx=%ld (>= K, multiple of 8) ldo=%ld (>= N)", who, ldx, ldo);
    if (M == 0) return 0;
    SMH_REQUIRE(x && w && out, "%s: null pointer", who);
    SMH_REQUIRE(((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0 && ((uintptr_t)out & 1) == 0, "%s: x and w must be 16-byte aligned", who);
    SMH_REQUIRE((long)M * ldx * 2 < (1L << 32) && (long)HEAD_BN * K * 2 < (1L << 32), "%s: lane offsets are 32-bit (M * ldx or 128 * K too large)", who);
    SMH_REQUIRE((M + HEAD_BM - 1) / HEAD_BM <= 65535, "%s: M=%d too large for one launch", who, M);
    static const head_kernel_t kern[9] = {nullptr, f16_head_kernel<1>, f16_head_kernel<2>, f16_head_kernel<3>, f16_head_kernel<4>,
                                          f16_head_kernel<5>, f16_head_kernel<6>, f16_head_kernel<7>, f16_head_kernel<8>};
    // more than 64 KB of dynamic LDS has to be allowed once per kernel (not stream work: fine under graph capture)
    static const hipError_t lds_ok = [] {
        hipError_t e = hipSuccess;
        for (int t = 1; t <= 8 && e == hipSuccess; ++t)
            e = hipFuncSetAttribute((const void *)kern[t], hipFuncAttributeMaxDynamicSharedMemorySize, head_stages(t) * (HEAD_W_BYTES + t * 16 * 128));
        return e;
    }();
    if (lds_ok != hipSuccess) { set_error("%s: hipFuncSetAttribute: %s", who, hipGetErrorString(lds_ok)); return (int)lds_ok; }
    HeadParams p;
    p.x = (const half_t *)x; p.w = (const half_t *)w; p.out = (half_t *)out;
    p.ldx = ldx; p.ldo = ldo; p.M = M; p.N = N; p.K = K;
    p.vec_store = (ldo % 4 == 0) && (((uintptr_t)out & 7) == 0);
    const int tiles = M >= HEAD_BM ? 8 : (M + 15) / 16;
    const size_t lds = (size_t)head_stages(tiles) * (HEAD_W_BYTES + tiles * 16 * 128);
    dim3 grid((unsigned)((N + HEAD_BN - 1) / HEAD_BN), (unsigned)((M + HEAD_BM - 1) / HEAD_BM));
    hipLaunchKernelGGL(kern[tiles], grid, dim3(HEAD_WAVES * 64), lds, (hipStream_t)stream, p);
    return launch_status();
}

extern "C" int smh_embedding(const int64_t *tokens, int M, const void *table, int vocab, int dim, void *out, smh_stream_t stream) {
    SMH_REQUIRE(M >= 0 && vocab > 0 && dim > 0 && dim % 8 == 0, "smh_embedding: M=%d vocab=%d dim=%d (dim must be a multiple of 8)", M, vocab, dim);
    if (M == 0) return 0;
    SMH_REQUIRE(tokens && table && out, "smh_embedding: null pointer");
    SMH_REQUIRE(((uintptr_t)table & 15) == 0 && ((uintptr_t)out & 15) == 0, "smh_embedding: table and out must be 16-byte aligned");
    hipLaunchKernelGGL(embedding_kernel, dim3((unsigned)M), dim3(256), 0, (hipStream_t)stream, tokens, (const half_t *)table, (half_t *)out, dim, vocab);
    return launch_status();
}
