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
// blockIdx.x = slice * units_pad + slot with units_pad a multiple of 8: workgroups are dealt round-robin
// to the 8 XCDs, so all K-slices of a column unit run behind the same L2, and slot -> unit gives every
// XCD a contiguous run of units (they share the cache lines of the scales).
#include "q40_matmul.hpp"
#include "slab_sum.hpp"

namespace smh {

constexpr int GEMV_COLS = 256;             // columns per workgroup
constexpr int GEMV_WAVES = 4;              // waves per workgroup, each with its own ring

// ---- per-wave ring of 32-row steps in LDS ----------------------------------------------------------
// The loads of a step go straight from global memory to LDS (global_load_lds, no VGPRs held while
// they are in flight): 4 x 1 KB of packed nibbles (8 rows x 128 B each), the step's 32 x 4 scales
// and the 16 x 32 tile of activations.  A wave keeps RING_STAGES steps in flight,
// which is what hides the HBM latency; it needs no barrier in its main loop because the ring is
// private to the wave (vmcnt orders the DMA against the wave's own LDS reads).
// Two stages: with the tiled layout (one contiguous 4352-byte run per stage) a third stage in flight per wave
// measured 1.5 % slower per launch and 2 % slower per decode step than two (eight waves a CU keep 16 stages,
// 70 KB, in flight either way the memory system's ~24 GB/s per CU share needs); four stages leave one workgroup a CU.
constexpr int RING_STAGES = 2;
constexpr int STAGE_W_BYTES = 32 * 128;
constexpr int STAGE_S_BYTES = 32 * 8;
constexpr int STAGE_X_BYTES = 16 * 64;
constexpr int STAGE_BYTES = STAGE_W_BYTES + STAGE_S_BYTES + STAGE_X_BYTES;   // 5376
constexpr int RING_BYTES = RING_STAGES * STAGE_BYTES;                        // 10752 per wave
// kernels that keep their activations in LDS outside the ring (LAYOUT 2 and 3) have no activation tile in a stage
constexpr int STAGE_BYTES_NO_X = STAGE_W_BYTES + STAGE_S_BYTES;             // 4352
constexpr int RING_BYTES_NO_X = RING_STAGES * STAGE_BYTES_NO_X;             // 8704 per wave

typedef const __attribute__((address_space(1))) void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;

struct GemvLane {
    const uint8_t *w_base;   // uniform: row 0 of this workgroup's 128-byte column
    const uint8_t *s_base;   // uniform: row 0 of its scales
    const uint8_t *x_base;   // uniform: the activations
    uint32_t w_off, s_off, x_off;   // this lane's byte offsets inside a step
    long w_row, s_row;       // row pitches in bytes
    int K, lane;
    bool two_blocks;
    int m_row;
};

// 6 vector-memory instructions per step.  For a full step the address is a uniform base (scalar
// registers, advanced by scalar arithmetic) plus a per-lane offset that never changes; only the
// last step of a K that is not a multiple of 32 clamps rows per lane.
template <bool RAGGED>
__device__ __forceinline__ void gemv_issue(const GemvLane &L, uint8_t *stage, int step) {
    const int k0 = step * 32;
    if constexpr (!RAGGED) {
        const uint8_t *wb = L.w_base + (long)k0 * L.w_row;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            __builtin_amdgcn_global_load_lds((gptr_t)(wb + (long)(8 * j) * L.w_row + L.w_off), (lptr_t)(stage + j * 1024), 16, 0, 0);
        // lane -> (row = lane / 2, block = lane % 2): one dword = (scale of columns 0..63, 64..127) of that block
        __builtin_amdgcn_global_load_lds((gptr_t)(L.s_base + (long)k0 * L.s_row + L.s_off), (lptr_t)(stage + STAGE_W_BYTES), 4, 0, 0);
        // lane -> (batch row = lane / 4, 8 k-values at 8 * (lane % 4))
        __builtin_amdgcn_global_load_lds((gptr_t)(L.x_base + 2 * k0 + L.x_off), (lptr_t)(stage + STAGE_W_BYTES + STAGE_S_BYTES), 16, 0, 0);
    } else {
        const int lane = L.lane;
        const int chunk = L.two_blocks ? (lane & 7) : (lane & 3);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = min(k0 + 8 * j + (lane >> 3), L.K - 1);
            __builtin_amdgcn_global_load_lds((gptr_t)(L.w_base + (long)row * L.w_row + 16 * chunk), (lptr_t)(stage + j * 1024), 16, 0, 0);
        }
        {
            const int row = min(k0 + (lane >> 1), L.K - 1);
            __builtin_amdgcn_global_load_lds((gptr_t)(L.s_base + (long)row * L.s_row + (L.two_blocks ? 4 * (lane & 1) : 0)),
                                             (lptr_t)(stage + STAGE_W_BYTES), 4, 0, 0);
        }
        {
            const int col = min(k0 + 8 * (lane & 3), L.K - 8);
            __builtin_amdgcn_global_load_lds((gptr_t)(L.x_base + (long)L.m_row + 2 * col), (lptr_t)(stage + STAGE_W_BYTES + STAGE_S_BYTES), 16, 0, 0);
        }
    }
}

// Tiled weights: the step's tile is one contiguous run of TILE_BYTES; lane l moves bytes 16 l .. 16 l + 15 of
// each 1 KB piece and dword l of the scales.  RAGGED only concerns the activations (rows of the tile past K
// hold zeros): their columns are clamped to stay inside the row.
template <bool RAGGED, bool WITH_A>
__device__ __forceinline__ void gemv_issue_tiled(const GemvLane &L, uint8_t *stage, int step) {
    const uint8_t *tile = L.w_base + (long)step * TILE_BYTES;
#pragma unroll
    for (int j = 0; j < 4; ++j)
        __builtin_amdgcn_global_load_lds((gptr_t)(tile + j * 1024 + L.w_off), (lptr_t)(stage + j * 1024), 16, 0, 0);
    __builtin_amdgcn_global_load_lds((gptr_t)(tile + TILE_W_BYTES + L.s_off), (lptr_t)(stage + STAGE_W_BYTES), 4, 0, 0);
    if constexpr (!WITH_A) return;
    const int k0 = step * 32;
    if constexpr (!RAGGED) {
        __builtin_amdgcn_global_load_lds((gptr_t)(L.x_base + 2 * k0 + L.x_off), (lptr_t)(stage + STAGE_W_BYTES + STAGE_S_BYTES), 16, 0, 0);
    } else {
        const int col = min(k0 + 8 * (L.lane & 3), L.K - 8);
        __builtin_amdgcn_global_load_lds((gptr_t)(L.x_base + (long)L.m_row + 2 * col), (lptr_t)(stage + STAGE_W_BYTES + STAGE_S_BYTES), 16, 0, 0);
    }
}

// The two masks, the two fp16 magic numbers and the two offsets of the decoder, held in registers the compiler cannot
// see through: (bits & mask) | magic then becomes ONE v_and_or_b32 (that instruction takes no literal operands, so
// with visible constants the compiler emits an AND and an OR).
struct GemvConsts {
    uint32_t mask_hi, mask_lo, magic_hi, magic_lo;
    h2 off_hi, off_lo;
};

// Decoding.  With u = nibble ^ 8 = code + 8:
//   high nibble: (bits & 0x00F0) | 0x5400 is the fp16 number 64 + u,   code = (64 + u) - 72     (exact)
//   low  nibble: (bits & 0x000F) | 0x6400 is the fp16 number 1024 + u, code = (1024 + u) - 1032 (exact)
// and ONE fp16 multiply by the group's scale gives the weight exactly as the reference's dequantiser rounds it,
// fp16(code * scale) (fp16_to_int4.py:90-96) - three packed instructions per two weights - which enters the matrix core as
// the B operand (lane = column, 8 consecutive k per lane) against the unscaled activations: the products the reference's
// kernel forms (triton_kernels.py:444-449), accumulated in fp32.
__device__ __forceinline__ uint32_t gemv_weights_high(uint32_t pr, h2 scale, const GemvConsts &C) {
    return as_u32((as_h2((pr & C.mask_hi) | C.magic_hi) + C.off_hi) * scale);
}
__device__ __forceinline__ uint32_t gemv_weights_low(uint32_t pr, h2 scale, const GemvConsts &C) {
    return as_u32((as_h2((pr & C.mask_lo) | C.magic_lo) + C.off_lo) * scale);
}

// acc[blk][h][b]: column 128*blk + 64*h + 4c + b.
template <bool RAGGED>
__device__ __forceinline__ void gemv_consume(const uint8_t *stage, int k0, int K, int c, int g, const GemvConsts &C,
                                             f4 (&acc)[2][2][4]) {
    uint32_t u0[8], u1[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        u0[i] = *reinterpret_cast<const uint32_t *>(stage + (8 * g + i) * 128 + 4 * c) ^ NIBBLE_FLIP;
        u1[i] = *reinterpret_cast<const uint32_t *>(stage + (8 * g + i) * 128 + 64 + 4 * c) ^ NIBBLE_FLIP;
    }
    h8 xv = *reinterpret_cast<const h8 *>(stage + STAGE_W_BYTES + STAGE_S_BYTES + c * 64 + 16 * g);
    if constexpr (RAGGED) {
        if (k0 + 8 * g >= K) {
#pragma unroll
            for (int i = 0; i < 8; ++i) xv[i] = (half_t)0.f;
        }
    }
    // scales of this lane's 8 rows: sv[i] = ((hi, lo) of block 0, (hi, lo) of block 1), regrouped per (block, half)
    // into the row pairs (2j, 2j+1) of the B operands
    u32x2 sv[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) sv[i] = *reinterpret_cast<const u32x2 *>(stage + STAGE_W_BYTES + (8 * g + i) * 8);
    h2 sc[2][2][4];
#pragma unroll
    for (int blk = 0; blk < 2; ++blk)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            sc[blk][0][j] = as_h2(pack_lo16(sv[2 * j][blk], sv[2 * j + 1][blk]));
            sc[blk][1][j] = as_h2(pack_hi16(sv[2 * j][blk], sv[2 * j + 1][blk]));
        }
#define SMH_GEMV_BYTE(U, BLK, B)                                                                 \
    {                                                                                            \
        u32x4 vh, vl;                                                                            \
        _Pragma("unroll") for (int j = 0; j < 4; ++j) {                                          \
            const uint32_t pr = pair_bytes<B>(U[2 * j], U[2 * j + 1]);                           \
            vh[j] = gemv_weights_high(pr, sc[BLK][0][j], C);                                     \
            vl[j] = gemv_weights_low(pr, sc[BLK][1][j], C);                                      \
        }                                                                                        \
        acc[BLK][0][B] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xv, __builtin_bit_cast(h8, vh), acc[BLK][0][B], 0, 0, 0);     \
        acc[BLK][1][B] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xv, __builtin_bit_cast(h8, vl), acc[BLK][1][B], 0, 0, 0);     \
    }
    SMH_GEMV_BYTE(u0, 0, 0)
    SMH_GEMV_BYTE(u0, 0, 1)
    SMH_GEMV_BYTE(u0, 0, 2)
    SMH_GEMV_BYTE(u0, 0, 3)
    SMH_GEMV_BYTE(u1, 1, 0)
    SMH_GEMV_BYTE(u1, 1, 1)
    SMH_GEMV_BYTE(u1, 1, 2)
    SMH_GEMV_BYTE(u1, 1, 3)
#undef SMH_GEMV_BYTE
}

// The same products from a tile (q40_matmul.hpp): the lane's 64 bytes are four linear 16-byte reads, the row
// pairs come out of (x, x2, x >> 8, x2 >> 8) and the scales arrive in the order of the row pairs.
// Same operands into the same MFMAs in the same order as gemv_consume: the results are bit-identical.
// `xrow`: the 8 activations k0 + 8g .. of this lane's batch row when they do not come from the stage (nullptr otherwise)
template <bool RAGGED, bool XROW = false>
__device__ __forceinline__ void gemv_consume_tiled(const uint8_t *stage, int k0, int K, int lane, const GemvConsts &C,
                                                   f4 (&acc)[2][2][4], const half_t *xrow = nullptr) {
    const int c = lane & 15, g = lane >> 4;
    u32x4 wq[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) wq[q] = *reinterpret_cast<const u32x4 *>(stage + q * 1024 + lane * 16);
    h8 xv;
    if constexpr (XROW) xv = *reinterpret_cast<const h8 *>(xrow);      // (no select between two pointers: this stays an LDS read)
    else xv = *reinterpret_cast<const h8 *>(stage + STAGE_W_BYTES + STAGE_S_BYTES + c * 64 + 16 * g);
    if constexpr (RAGGED) {
        if (k0 + 8 * g >= K) {
#pragma unroll
            for (int i = 0; i < 8; ++i) xv[i] = (half_t)0.f;
        }
    }
    // sc[grp][j]: scales of rows (2j, 2j+1) of this lane's k-octet for the unit's 64-column group grp = 2 blk + half
    u32x4 sc[4];
#pragma unroll
    for (int grp = 0; grp < 4; ++grp) sc[grp] = *reinterpret_cast<const u32x4 *>(stage + STAGE_W_BYTES + g * 64 + grp * 16);
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int blk = q >> 1, B = 2 * (q & 1) + half;
            const uint32_t pr[4] = {wq[q][2 * half], wq[q][2 * half + 1], wq[q][2 * half] >> 8, wq[q][2 * half + 1] >> 8};
            u32x4 vh, vl;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                vh[j] = gemv_weights_high(pr[j], as_h2(sc[2 * blk][j]), C);
                vl[j] = gemv_weights_low(pr[j], as_h2(sc[2 * blk + 1][j]), C);
            }
            acc[blk][0][B] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xv, __builtin_bit_cast(h8, vh), acc[blk][0][B], 0, 0, 0);
            acc[blk][1][B] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xv, __builtin_bit_cast(h8, vl), acc[blk][1][B], 0, 0, 0);
        }
}

// LAYOUT 0: checkpoint layout; 1: tiled weights (smh_q40_tile); 2: tiled weights and activations made from the
// gate|up slabs by the workgroup itself (p.gu_partial): SiLU(gate) * up needs no launch of its own; 3: tiled weights
// and activations made from the residual stream by the workgroup itself (p.norm_w, p.norm_ss): RMSNorm needs only
// the small launch that adds the slabs and leaves the sums of squares
template <int LAYOUT>
__global__ __launch_bounds__(GEMV_WAVES * 64) void q40_gemv_kernel(MatmulParams p) {
    constexpr int WAVES = GEMV_WAVES;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];   // WAVES rings, then reused as red[WAVES][M][256]
    constexpr int THREADS = WAVES * 64;
    constexpr bool TILED = LAYOUT != 0;
    constexpr bool SILU_IN = LAYOUT == 2;
    constexpr bool NORM_IN = LAYOUT == 3;
    constexpr bool X_IN_LDS = SILU_IN || NORM_IN;                   // activations: xs[M][slice rows] behind the rings
    constexpr int PER_STAGE = X_IN_LDS ? 5 : 6;                     // vector-memory instructions per stage
    constexpr int STAGE = X_IN_LDS ? STAGE_BYTES_NO_X : STAGE_BYTES;
    constexpr int RING = RING_STAGES * STAGE;

    // Workgroups are dealt round-robin to the 8 XCDs (8 L2s).  Neighbouring column units share the 128-byte
    // lines of the scale rows, so each XCD takes a CONTIGUOUS run of units: a scale line is then fetched
    // from HBM by one L2, not by eight.
    const int slot = blockIdx.x % p.units_pad;
    const int unit = (slot & 7) * (p.units_pad >> 3) + (slot >> 3);
    const int slice = blockIdx.x / p.units_pad;
    if (unit >= p.units) return;
    // which segment (weight) does this column pair belong to
    int sg = 0;
    if (p.nseg > 1 && unit >= p.seg[1].unit0) sg = 1;
    if (p.nseg > 2 && unit >= p.seg[2].unit0) sg = 2;
    const MatmulSegment seg = p.seg[sg];
    const int pair = unit - seg.unit0;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int c = lane & 15;
    const int g = lane >> 4;
    const int col0 = pair * GEMV_COLS;     // first column (inside the segment) of this workgroup
    // when N/128 is odd the last pair has no second block: its loads re-read the first block (valid
    // memory) and the results of those columns are dropped
    const bool two_blocks = col0 + 128 < seg.N;

    GemvLane L;
    L.K = p.K;
    L.lane = lane;
    L.two_blocks = two_blocks;
    L.w_row = seg.N / 2;
    L.s_row = seg.N / 32;
    L.w_base = seg.w + (long)pair * 128;
    L.s_base = reinterpret_cast<const uint8_t *>(seg.s) + (long)pair * 8;
    L.x_base = reinterpret_cast<const uint8_t *>(p.a);
    L.m_row = (int)(min(lane >> 2, p.M - 1) * p.lda * 2);
    L.w_off = (uint32_t)((lane >> 3) * (seg.N / 2) + 16 * (two_blocks ? (lane & 7) : (lane & 3)));
    L.s_off = (uint32_t)((lane >> 1) * (seg.N / 32) + (two_blocks ? 4 * (lane & 1) : 0));
    L.x_off = (uint32_t)(L.m_row + 16 * (lane & 3));
    if constexpr (TILED) {
        L.w_base = seg.w + (long)pair * tiled_steps(p.K) * TILE_BYTES;     // this unit's tiles, step 0
        L.w_off = (uint32_t)(16 * lane);
        L.s_off = (uint32_t)(4 * lane);
    }
    uint8_t *ring = lds + wave * RING;

    GemvConsts C{0x00F000F0u, 0x000F000Fu, 0x54005400u, 0x64006400u, h2{(half_t)-72.f, (half_t)-72.f}, h2{(half_t)-1032.f, (half_t)-1032.f}};
    asm volatile("" : "+s"(C.mask_hi), "+s"(C.mask_lo));
    asm volatile("" : "+v"(C.magic_hi), "+v"(C.magic_lo));

    f4 acc[2][2][4];
#pragma unroll
    for (int d = 0; d < 2; ++d)
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int b = 0; b < 4; ++b) acc[d][h][b] = f4{0.f, 0.f, 0.f, 0.f};

    // this wave's steps: first, first + WAVES, ...
    const int step0 = slice * p.steps_per_slice;
    const int step1 = min(step0 + p.steps_per_slice, (p.K + 31) / 32);
    const int first = step0 + wave;
    const int n_steps = first < step1 ? (step1 - first + WAVES - 1) / WAVES : 0;
    const int full_steps = p.K / 32;        // steps below this index have all their 32 rows
    auto issue = [&](uint8_t *stage, int step) {
        if constexpr (TILED) {
            if (step < full_steps) gemv_issue_tiled<false, !X_IN_LDS>(L, stage, step);
            else gemv_issue_tiled<true, !X_IN_LDS>(L, stage, step);
        } else {
            if (step < full_steps) gemv_issue<false>(L, stage, step);
            else gemv_issue<true>(L, stage, step);
        }
    };
    // SILU_IN: xs[M][slice rows] fp16 behind the rings.  The slab loads of this thread's share are requested first, the
    // weight stages right behind them, so that both are in flight together.
    half_t *xs = reinterpret_cast<half_t *>(lds + WAVES * RING);
    const int slice_k0 = step0 * 32, slice_rows = (step1 - step0) * 32;
    // a row of xs is 16 bytes longer than its data: the 16 lanes that read one k-octet of 16 different rows would
    // otherwise hit the same LDS banks whenever the slice is a multiple of 128 bytes long
    const int xs_pitch = slice_rows + 8;
    if constexpr (SILU_IN) {
        constexpr int MAXQ = SMH_SILU_IN_MAX_M * SMH_SILU_IN_MAX_K / 4 / THREADS;     // quads of columns per thread
        f4 ga[MAXQ], ua[MAXQ];
        const int quads = slice_rows / 4, total = p.M * quads;
        const long gu_slab = (long)p.M * 2 * p.K;
        // item idx = (row idx / quads, quad idx % quads); idx < 1024, so the quotient from a float reciprocal is exact
        const float inv_quads = 1.0f / (float)max(quads, 1);
        auto row_of = [&](int idx) { return (int)(((float)idx + 0.5f) * inv_quads); };
#pragma unroll
        for (int i = 0; i < MAXQ; ++i) {
            const int idx = tid + i * THREADS;
            if (idx < total) {
                const int m = row_of(idx), k = slice_k0 + 4 * (idx - m * quads);
                if (k < p.K) {
                    ga[i] = slab_sum4(p.gu_partial, (long)m * 2 * p.K + k, gu_slab, p.gu_ksplit);
                    ua[i] = slab_sum4(p.gu_partial, (long)m * 2 * p.K + p.K + k, gu_slab, p.gu_ksplit);
                } else {
                    ga[i] = f4{0.f, 0.f, 0.f, 0.f};
                    ua[i] = f4{0.f, 0.f, 0.f, 0.f};
                }
            }
        }
#pragma unroll
        for (int i = 0; i < RING_STAGES; ++i)
            if (i < n_steps) issue(ring + i * STAGE, first + i * WAVES);
#pragma unroll
        for (int i = 0; i < MAXQ; ++i) {
            const int idx = tid + i * THREADS;
            if (idx < total) {
                h4 o;
#pragma unroll
                for (int j = 0; j < 4; ++j) {                  // the roundings of partial_silu_mul_kernel
                    const float gf = (float)(half_t)ga[i][j];
                    const half_t sl = (half_t)(gf / (1.0f + expf(-gf)));
                    o[j] = sl * (half_t)ua[i][j];
                }
                const int m = row_of(idx);
                *reinterpret_cast<h4 *>(xs + (long)m * xs_pitch + 4 * (idx - m * quads)) = o;
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");      // xs is complete; the DMA ring stays in flight
    } else if constexpr (NORM_IN) {
        // the loads of this thread's share of h (eight consecutive k of one row at a time), of the matching norm
        // weights and, in the first threads, of a row's sums of squares go out first, the weight stages right
        // behind them
        constexpr int MAXO = (SMH_NORM_IN_MAX_XS_BYTES / 16 + THREADS - 1) / THREADS;     // k-octets per thread
        float *s_r = reinterpret_cast<float *>(xs + (long)p.M * xs_pitch);           // r[m], behind xs
        h8 hv[MAXO], wv[MAXO];
        const int octs = slice_rows / 8, total = p.M * octs;
        // item idx = (row idx / octs, octet idx % octs); idx < 1760 and octs <= 1760, so the quotient from a float
        // reciprocal is exact (an integer division costs ~25 instructions per item here)
        const float inv_octs = 1.0f / (float)max(octs, 1);
        auto row_of = [&](int idx) { return (int)(((float)idx + 0.5f) * inv_octs); };
#pragma unroll
        for (int i = 0; i < MAXO; ++i) {
            const int idx = tid + i * THREADS;
            if (idx < total) {
                const int m = row_of(idx), k = slice_k0 + 8 * (idx - m * octs);
                if (k < p.K) {
                    hv[i] = *reinterpret_cast<const h8 *>(p.a + (long)m * p.lda + k);
                    wv[i] = *reinterpret_cast<const h8 *>(p.norm_w + k);
                } else {
                    hv[i] = h8{0, 0, 0, 0, 0, 0, 0, 0};
                    wv[i] = hv[i];
                }
            }
        }
        f4 ssv[SMH_NORM_SUMS / 4];
        if (tid < p.M) {
#pragma unroll
            for (int j = 0; j < SMH_NORM_SUMS / 4; ++j) ssv[j] = *reinterpret_cast<const f4 *>(p.norm_ss + (long)tid * SMH_NORM_SUMS + 4 * j);
        }
#pragma unroll
        for (int i = 0; i < RING_STAGES; ++i)
            if (i < n_steps) issue(ring + i * STAGE, first + i * WAVES);
        if (tid < p.M) {
            float sum = 0.f;
#pragma unroll
            for (int j = 0; j < SMH_NORM_SUMS; ++j) sum += ssv[j / 4][j % 4];
            s_r[tid] = rms_factor(sum, p.K, p.norm_eps);
        }
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");      // r[] is complete
#pragma unroll
        for (int i = 0; i < MAXO; ++i) {
            const int idx = tid + i * THREADS;
            if (idx < total) {
                const int m = row_of(idx);
                const float r = s_r[m];
                h8 o;
#pragma unroll
                for (int j = 0; j < 8; ++j) {                  // the roundings of partial_rmsnorm_kernel
                    const half_t nv = scale_to_half(hv[i][j], r);
                    o[j] = nv * wv[i][j];
                }
                *reinterpret_cast<h8 *>(xs + (long)m * xs_pitch + 8 * (idx - m * octs)) = o;
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");      // xs is complete; the DMA ring stays in flight
    } else {
#pragma unroll
        for (int i = 0; i < RING_STAGES; ++i)
            if (i < n_steps) issue(ring + i * STAGE, first + i * WAVES);
    }
    const half_t *xlane = xs + (long)min(c, p.M - 1) * xs_pitch + 8 * g;     // X_IN_LDS: this lane's row of xs, its k-octet
    // the one step that may lack rows is the last step of K, hence the last one of its wave; it is
    // peeled off so that the loop has a single decoder in it
    const int n_full = first < full_steps ? min(n_steps, (full_steps - first + WAVES - 1) / WAVES) : 0;
    int stage = 0;
    for (int i = 0; i < n_full; ++i) {
        const int later = min(RING_STAGES - 1, n_steps - 1 - i);     // steps issued after step i and still in flight
        if (later >= 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * PER_STAGE) : "memory");
        else if (later == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(PER_STAGE) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if constexpr (X_IN_LDS) gemv_consume_tiled<false, true>(ring + stage * STAGE, 0, p.K, lane, C, acc, xlane + (first + i * WAVES - step0) * 32);
        else if constexpr (TILED) gemv_consume_tiled<false>(ring + stage * STAGE, 0, p.K, lane, C, acc);
        else gemv_consume<false>(ring + stage * STAGE, 0, p.K, c, g, C, acc);
        if (i + RING_STAGES < n_steps) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");        // this stage's LDS reads are done
            issue(ring + stage * STAGE, first + (i + RING_STAGES) * WAVES);
        }
        stage = (stage + 1 == RING_STAGES) ? 0 : stage + 1;
    }
    if (n_full < n_steps) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if constexpr (X_IN_LDS) gemv_consume_tiled<true, true>(ring + stage * STAGE, (first + n_full * WAVES) * 32, p.K, lane, C, acc, xlane + (first + n_full * WAVES - step0) * 32);
        else if constexpr (TILED) gemv_consume_tiled<true>(ring + stage * STAGE, (first + n_full * WAVES) * 32, p.K, lane, C, acc);
        else gemv_consume<true>(ring + stage * STAGE, (first + n_full * WAVES) * 32, p.K, c, g, C, acc);
    }
    __syncthreads();                        // every wave is done with its ring: reuse LDS for the sums

    // ---- add the waves' partial sums through LDS ----
    // accumulator element r of acc[blk][h][b] in lane (g, c) is row m = 4g + r,
    // column 128*blk + 64h + 4c + b of the workgroup's 256
    float *red = reinterpret_cast<float *>(lds);
#pragma unroll
    for (int d = 0; d < 2; ++d)
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = 4 * g + r;
                if (r < p.M) {                      // uniform: with fewer than 4 rows whole store instructions drop out
                    if (m < p.M) {                  // the four columns 4c .. 4c+3 of (block d, half h) as one 16-byte store
                        *reinterpret_cast<f4 *>(&red[(wave * p.M + m) * GEMV_COLS + 128 * d + 64 * h + 4 * c]) =
                            f4{acc[d][h][0][r], acc[d][h][1][r], acc[d][h][2][r], acc[d][h][3][r]};
                    }
                }
            }
    __syncthreads();

    const int outputs = p.M * GEMV_COLS;
    float *slab = p.partial + (long)slice * p.M * p.n_total;
    if (!p.direct) {
        // slabs: four consecutive columns per thread (segment widths are multiples of 128, so a quad is inside or outside)
        for (int q = tid; q < outputs / 4; q += THREADS) {
            f4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int wv_ = 0; wv_ < WAVES; ++wv_) sum += *reinterpret_cast<const f4 *>(red + wv_ * outputs + 4 * q);
            const int m = q >> 6, n_seg = col0 + 4 * (q & 63);
            if (n_seg < seg.N) *reinterpret_cast<f4 *>(slab + (long)m * p.n_total + seg.col0 + n_seg) = sum;
        }
        return;
    }
    // thread -> outputs idx = tid, tid + THREADS, ... with idx = m * 256 + local column
    for (int idx = tid; idx < outputs; idx += THREADS) {
        float sum = 0.f;
#pragma unroll
        for (int wv_ = 0; wv_ < WAVES; ++wv_) sum += red[wv_ * outputs + idx];
        const int m = idx >> 8, n_seg = col0 + (idx & 255);
        if (n_seg >= seg.N) continue;
        const int n = seg.col0 + n_seg;
        p.c[(long)m * p.ldc + n] = matmul_epilogue(p, sum, m, n);
    }
}

}  // namespace smh

namespace smh {

// K is cut into slices so that the launch fills the GPU in ONE round of workgroups: two
// workgroups (two sets of LDS rings) fit a CU, 256 CUs, so at most 512 workgroups; a launch of a
// few more than that would run a second, nearly empty round and take twice as long.
void gemv_plan(int n_total_units, int K, int waves, int *ksplit, int *steps_per_slice) {
    const int steps = (K + 31) / 32;
    constexpr int capacity = 512;
    int ks = capacity / n_total_units;              // floor: never exceed one round
    if (ks < 1) ks = 1;
    if (ks > SMH_MAX_KSPLIT) ks = SMH_MAX_KSPLIT;
    int max_split = (steps + waves - 1) / waves;    // every wave should have a step
    if (ks > max_split) ks = max_split;
    const int sps = (steps + ks - 1) / ks;
    *ksplit = (steps + sps - 1) / sps;
    *steps_per_slice = sps;
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
    gemv_plan(p.units, p.K, GEMV_WAVES, &p.ksplit, &p.steps_per_slice);
}

bool gemv_norm_in_fits(const MatmulParams &p) {
    return p.M <= SMH_GEMV_MAX_M && (size_t)p.M * (p.steps_per_slice * 32 + 8) * sizeof(half_t) <= SMH_NORM_IN_MAX_XS_BYTES;
}

int gemv_launch(const MatmulParams &p, hipStream_t stream) {
    constexpr int waves = GEMV_WAVES;
    dim3 grid((unsigned)(p.units_pad * p.ksplit));
    size_t lds = (size_t)waves * RING_BYTES;                       // rings, reused for the [waves][M][256] sums
    const size_t red = (size_t)waves * p.M * GEMV_COLS * sizeof(float);
    if (p.tiled && (p.gu_partial != nullptr || p.norm_w != nullptr))   // rings without activation tiles, xs (and r[]) behind them
        lds = (size_t)waves * RING_BYTES_NO_X + (size_t)p.M * (p.steps_per_slice * 32 + 8) * sizeof(half_t) + SMH_GEMV_MAX_M * sizeof(float);
    if (red > lds) lds = red;
    if (p.tiled) {
        if (p.gu_partial != nullptr) {
            if (p.M > SMH_SILU_IN_MAX_M || p.steps_per_slice * 32 > SMH_SILU_IN_MAX_K) {
                set_error("q40 gemv: activations from the gate|up slabs need M <= %d and K-slices of at most %d rows", SMH_SILU_IN_MAX_M,
                          SMH_SILU_IN_MAX_K);
                return -1;
            }
            // more than 64 KB of dynamic LDS has to be allowed once (not stream work: fine under graph capture)
            static const hipError_t lds_ok = hipFuncSetAttribute((const void *)q40_gemv_kernel<2>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                                                 80 * 1024);
            if (lds_ok != hipSuccess) {
                set_error("q40 gemv: the kernel's LDS could not be reserved: %s", hipGetErrorString(lds_ok));
                return (int)lds_ok;
            }
            hipLaunchKernelGGL((q40_gemv_kernel<2>), grid, dim3(256), lds, stream, p);
        } else if (p.norm_w != nullptr) {
            if (!gemv_norm_in_fits(p)) {
                set_error("q40 gemv: %d rows x K-slices of %d rows do not fit next to the weight rings (RMSNorm inside the matmul)", p.M,
                          p.steps_per_slice * 32);
                return -1;
            }
            static const hipError_t lds_ok = hipFuncSetAttribute((const void *)q40_gemv_kernel<3>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                                                 80 * 1024);
            if (lds_ok != hipSuccess) {
                set_error("q40 gemv: the kernel's LDS could not be reserved: %s", hipGetErrorString(lds_ok));
                return (int)lds_ok;
            }
            hipLaunchKernelGGL((q40_gemv_kernel<3>), grid, dim3(256), lds, stream, p);
        } else {
            hipLaunchKernelGGL((q40_gemv_kernel<1>), grid, dim3(256), lds, stream, p);
        }
    } else {
        hipLaunchKernelGGL((q40_gemv_kernel<0>), grid, dim3(256), lds, stream, p);
    }
    return launch_status();
}

}  // namespace smh
