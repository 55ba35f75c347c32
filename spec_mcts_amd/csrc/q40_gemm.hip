// Q4_0 dequant + matmul for large batches (decode at B = 100, prefill): c[M,N] = a[M,K] . deq(W)[K,N].
//
// A workgroup of 4 waves (8 on tiled weights, plus one that only issues DMA in launches with one workgroup per compute
// unit, see the kernel) owns 128 rows of A, two adjacent 128-column blocks of the weight (one full 128-byte line of
// packed nibbles per k) and a slice of K - or, under a range cut, a run of steps that may end one column unit and begin
// the next; up to two workgroups share a compute unit.  Everything a 32-row step needs - 4 KB of nibbles, 256 B of scales, the 128 x 32 tile of A -
// goes global -> LDS by DMA (global_load_lds) into a 6-slot ring shared by the workgroup; one bare s_barrier
// per TWO steps both publishes stages and frees the oldest ones.  (__syncthreads() would wait for every
// outstanding DMA first, because they write LDS, and so empty the ring at every barrier.)
//   * wave w decodes TWO byte positions of ONE block (block w/2, bytes 2(w%2) and 2(w%2)+1 of every
//     dword): perm pairs the byte of two consecutive rows, and-or drops the nibbles into fp16
//     mantissas, one packed op recovers the exact code and one packed multiply applies the scales -
//     the value the reference's dequantiser produces, born in the B-operand layout of
//     v_mfma_f32_16x16x32_f16, so dequantised weights never travel through LDS or HBM;
//   * it multiplies its four B operands (2 byte positions x high / low nibbles = columns c and c+64)
//     with all TILES 16-row tiles of A, read from LDS with an XOR swizzle that keeps ds_read_b128
//     conflict-free: one read of the A tile feeds four MFMAs;
//   * the step is software-pipelined inside the wave: while the matrix pipe works through step i,
//     the vector ALU decodes the B operands of step i+1 (one basic block, no branches: the number of
//     row tiles and the ragged-K handling are template parameters), and the DMA addresses are a
//     scalar base per step plus lane offsets that never change, so issuing a stage costs no VALU work;
//   * the accumulators leave through LDS one row tile at a time, so global stores are 64-byte
//     contiguous per lane; K-slices are written as fp32 slabs and added by the consuming kernel.
//
// At M = 100 the work sits on the ridge of the roofline: 2*M*N*K flops against
// N*K*0.53125 + 2*M*(K+N) bytes.
#include <type_traits>

#include "q40_matmul.hpp"

namespace smh {

// most K-slices of a launch = GEMM_KSCAP / rows (every slice leaves an fp32 slab of rows x columns)
constexpr int GEMM_KSCAP = 1600;
constexpr int GEMM_BM = 128;
constexpr int GEMM_WAVES = 4;                  // checkpoint layout and ragged K; tiled weights run GEMM_TILED_WAVES
constexpr int GEMM_TILED_WAVES = 8;
constexpr int GEMM_THREADS = GEMM_WAVES * 64;
// slots of the DMA ring (with a barrier per step, four slots measured 2 % faster per launch at M=100 than six; with a
// barrier per two steps, six slots are 3 % faster than that)
constexpr int GEMM_STAGES = 6;
// slots of the ring in the variant with a DMA wave (eight measured like six) and the most workgroups of a launch that
// takes it (one per compute unit)
constexpr int GEMM_DMA_WAVE_SLOTS = 6;
constexpr int GEMM_DMA_WAVE_MAX_WGS = 256;
constexpr int GS_WBLOCK = 8 * 128 + 64;        // the 8 rows one wave fetches, padded by 16 banks: the four row groups a
                                               // ds_read_b32 touches (lanes 16g..16g+15 read row 8g+r) then sit in different banks
constexpr int GS_W = 4 * GS_WBLOCK;            // nibbles
constexpr int GS_S = 32 * 8;                   // scales
constexpr int GS_A = GEMM_BM * 64;             // A tile, 64 B per row, 16-byte chunks XOR-swizzled
constexpr int GS_BYTES = GS_W + GS_S + GS_A;               // 12800
constexpr int GEMM_LDS = GEMM_STAGES * GS_BYTES;           // 76800
constexpr int GEMM_COLS = 256;

typedef const __attribute__((address_space(1))) void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;


// Waits until at most N DMA instructions of this wave are still in flight (the counter has six bits).
template <int N>
__device__ __forceinline__ void gemm_wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N < 63 ? N : 63) : "memory"); }
// ... at most `stages` younger stages of PER DMA instructions each (4 with four waves, 2 with eight, 5 + row tiles in
// the DMA wave).
template <int PER>
__device__ __forceinline__ void gemm_wait_dma(int stages) {
    switch (stages) {
        case 5: gemm_wait_vm<5 * PER>(); break;
        case 4: gemm_wait_vm<4 * PER>(); break;
        case 3: gemm_wait_vm<3 * PER>(); break;
        case 2: gemm_wait_vm<2 * PER>(); break;
        case 1: gemm_wait_vm<1 * PER>(); break;
        default: gemm_wait_vm<0>(); break;
    }
}

// A bare workgroup barrier.  Every LDS read this wave has issued has returned (lgkmcnt), so after the
// barrier no wave still reads the stage that is refilled next.
__device__ __forceinline__ void gemm_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// TILED: the weights are in the tiled layout (q40_matmul.hpp).  Wave w then moves and decodes piece w of a
// tile (its two byte positions of its block, already paired by rows): one 16-byte LDS read instead of eight
// dword reads, shifts instead of byte permutes, the scales already in operand order; rows past K hold zeros.
// WAVES = 8 (tiled weights only): waves w and w + 4 share piece w of a tile; wave w multiplies the columns of its HIGH
// nibbles, wave w + 4 those of the low nibbles (two B operands and half the accumulators each, the same A tiles), so
// that every SIMD holds two waves of the workgroup and the decode of one runs under the MFMAs of the other.
//
// One piece of a workgroup's work: steps [step0, step1) of column unit `unit` (row block mb), accumulated and left as slab
// `slice`.  zero_rest: the piece ends its unit, and the slabs past `slice` (the unit has no piece for them) are written as
// zeros.  more: another piece follows in this workgroup (one more barrier, after which the ring may be refilled).
// tid_bias: zero (a range cut passes one the compiler cannot see, see there).
template <int TILES, bool RAGGED, bool TILED, int WAVES, int SLOTS, bool PRODUCER>
__device__ __forceinline__ void gemm_piece(const MatmulParams &p, int unit, int mb, int slice, int step0, int step1, bool zero_rest, bool more,
                                           int tid_bias) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr int NB = WAVES == 8 ? 2 : 4;     // B operands (16 columns each) per wave
    constexpr int DMA_PER = WAVES == 8 ? 2 : 4;

    const int tid = threadIdx.x + tid_bias;
    const int wave8 = tid >> 6;                // 0 .. WAVES-1
    const int wave = wave8 & 3;                // piece of the tile / rows of the ring this wave serves
    const int hh = wave8 >> 2;                 // eight waves: 0 = high nibbles (columns c), 1 = low nibbles (columns c + 64)
    const int lane = tid & 63;
    const int c = lane & 15;
    const int g = lane >> 4;
    int sg = 0;
    if (p.nseg > 1 && unit >= p.seg[1].unit0) sg = 1;
    if (p.nseg > 2 && unit >= p.seg[2].unit0) sg = 2;
    const MatmulSegment seg = p.seg[sg];
    const int pair = unit - seg.unit0;
    const int col0 = pair * GEMM_COLS;
    const bool two_blocks = col0 + 128 < seg.N;
    const int m0 = mb * p.block_rows;
    const int blk = wave >> 1;                 // block of the pair this wave decodes
    const int bp = wave & 1;                   // ... and its pair of byte positions
    const uint32_t sel0 = 0x0c000c00u | (uint32_t)(2 * bp) | ((uint32_t)(4 + 2 * bp) << 16);
    const uint32_t sel1 = sel0 + 0x00010001u;

    const long w_row = seg.N / 2;              // bytes per k of the nibbles
    const long s_row = seg.N / 32;             // bytes per k of the scales
    // ---- this wave's four DMA instructions per stage ----
    //  rows 8w .. 8w+7 of the nibbles; their scales (lanes 0..15); rows 32w .. 32w+31 of the A tile.
    //  Address = uniform base of the step (scalar arithmetic) + a lane offset fixed for the whole kernel.
    const uint8_t *w_base = TILED ? seg.w + (long)pair * tiled_steps(p.K) * TILE_BYTES : seg.w + (long)pair * 128;
    const uint8_t *s_base = reinterpret_cast<const uint8_t *>(seg.s) + (long)pair * 8;
    const uint8_t *a_base = reinterpret_cast<const uint8_t *>(p.a);
    const int w_lrow = 8 * wave + (lane >> 3), w_lcol = 16 * (two_blocks ? (lane & 7) : (lane & 3));
    const int s_lrow = 8 * wave + ((lane & 15) >> 1), s_lcol = 4 * (two_blocks ? (lane & 1) : 0);
    const int a_chunk = (lane & 3) ^ ((lane >> 4) & 3);                   // logical 16-byte chunk stored in slot lane&3
    const long a_r0 = (long)min(m0 + (WAVES == 8 ? 16 * wave8 : 32 * wave) + (lane >> 2), p.M - 1) * p.lda * 2;
    const long a_r1 = (long)min(m0 + 32 * wave + 16 + (lane >> 2), p.M - 1) * p.lda * 2;
    const uint32_t w_voff = (uint32_t)(w_lrow * w_row + w_lcol);
    const uint32_t s_voff = (uint32_t)(s_lrow * s_row + s_lcol);
    const uint32_t a_voff0 = (uint32_t)(a_r0 + 16 * a_chunk), a_voff1 = (uint32_t)(a_r1 + 16 * a_chunk);

    // eight waves: the two DMA instructions of a wave and stage separately, so that the A rows' (no branch around it)
    // can go between the MFMAs of a step
    auto issue_ws8 = [&](int step, int slot_) {
        uint8_t *st = lds + slot_ * GS_BYTES;
        const uint8_t *tile = w_base + (long)step * TILE_BYTES;
        if (hh == 0) __builtin_amdgcn_global_load_lds((gptr_t)(tile + wave * 1024 + lane * 16), (lptr_t)(st + wave * 1024), 16, 0, 0);
        else if (lane < 16) __builtin_amdgcn_global_load_lds((gptr_t)(tile + TILE_W_BYTES + (16 * wave + lane) * 4), (lptr_t)(st + GS_W + wave * 64), 4, 0, 0);
    };
    auto issue_a8 = [&](int step, int slot_) {
        __builtin_amdgcn_global_load_lds((gptr_t)(a_base + (long)step * 64 + a_voff0), (lptr_t)(lds + slot_ * GS_BYTES + GS_W + GS_S + wave8 * 1024), 16, 0, 0);
    };
    auto issue = [&](int step, int slot_) {
        uint8_t *st = lds + slot_ * GS_BYTES;
        const long k0 = (long)step * 32;
        if (TILED && WAVES == 8) {
            // two DMA instructions a wave: waves 0-3 their piece of the nibbles, waves 4-7 its scales; every wave 16 rows of A
            const uint8_t *tile = w_base + (long)step * TILE_BYTES;
            if (hh == 0) __builtin_amdgcn_global_load_lds((gptr_t)(tile + wave * 1024 + lane * 16), (lptr_t)(st + wave * 1024), 16, 0, 0);
            else if (lane < 16) __builtin_amdgcn_global_load_lds((gptr_t)(tile + TILE_W_BYTES + (16 * wave + lane) * 4), (lptr_t)(st + GS_W + wave * 64), 4, 0, 0);
            __builtin_amdgcn_global_load_lds((gptr_t)(a_base + k0 * 2 + a_voff0), (lptr_t)(st + GS_W + GS_S + wave8 * 1024), 16, 0, 0);
        } else if (TILED) {
            const uint8_t *tile = w_base + (long)step * TILE_BYTES;
            __builtin_amdgcn_global_load_lds((gptr_t)(tile + wave * 1024 + lane * 16), (lptr_t)(st + wave * 1024), 16, 0, 0);
            if (lane < 16)
                __builtin_amdgcn_global_load_lds((gptr_t)(tile + TILE_W_BYTES + (16 * wave + lane) * 4), (lptr_t)(st + GS_W + wave * 64), 4, 0, 0);
            if (!RAGGED) {
                __builtin_amdgcn_global_load_lds((gptr_t)(a_base + k0 * 2 + a_voff0), (lptr_t)(st + GS_W + GS_S + wave * 2048), 16, 0, 0);
                __builtin_amdgcn_global_load_lds((gptr_t)(a_base + k0 * 2 + a_voff1), (lptr_t)(st + GS_W + GS_S + wave * 2048 + 1024), 16, 0, 0);
            } else {
                const long ac = min(k0 + 8 * a_chunk, (long)p.K - 8) * 2;
                __builtin_amdgcn_global_load_lds((gptr_t)(a_base + a_r0 + ac), (lptr_t)(st + GS_W + GS_S + wave * 2048), 16, 0, 0);
                __builtin_amdgcn_global_load_lds((gptr_t)(a_base + a_r1 + ac), (lptr_t)(st + GS_W + GS_S + wave * 2048 + 1024), 16, 0, 0);
            }
        } else if (!RAGGED) {
            __builtin_amdgcn_global_load_lds((gptr_t)(w_base + k0 * w_row + w_voff), (lptr_t)(st + wave * GS_WBLOCK), 16, 0, 0);
            if (lane < 16)
                __builtin_amdgcn_global_load_lds((gptr_t)(s_base + k0 * s_row + s_voff), (lptr_t)(st + GS_W + wave * 64), 4, 0, 0);
            __builtin_amdgcn_global_load_lds((gptr_t)(a_base + k0 * 2 + a_voff0), (lptr_t)(st + GS_W + GS_S + wave * 2048), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((gptr_t)(a_base + k0 * 2 + a_voff1), (lptr_t)(st + GS_W + GS_S + wave * 2048 + 1024), 16, 0, 0);
        } else {
            // rows past K repeat row K-1 (their products are masked out below); the A columns stay inside the row
            const long wr = min(k0 + w_lrow, (long)p.K - 1), sr = min(k0 + s_lrow, (long)p.K - 1);
            const long ac = min(k0 + 8 * a_chunk, (long)p.K - 8) * 2;
            __builtin_amdgcn_global_load_lds((gptr_t)(w_base + wr * w_row + w_lcol), (lptr_t)(st + wave * GS_WBLOCK), 16, 0, 0);
            if (lane < 16)
                __builtin_amdgcn_global_load_lds((gptr_t)(s_base + sr * s_row + s_lcol), (lptr_t)(st + GS_W + wave * 64), 4, 0, 0);
            __builtin_amdgcn_global_load_lds((gptr_t)(a_base + a_r0 + ac), (lptr_t)(st + GS_W + GS_S + wave * 2048), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((gptr_t)(a_base + a_r1 + ac), (lptr_t)(st + GS_W + GS_S + wave * 2048 + 1024), 16, 0, 0);
        }
    };

    f4 acc[NB][TILES];
#pragma unroll
    for (int h = 0; h < NB; ++h)
#pragma unroll
        for (int t = 0; t < TILES; ++t) acc[h][t] = f4{0.f, 0.f, 0.f, 0.f};

    const int n_steps = max(step1 - step0, 0);
    // workgroups that share a K-slice read the same A tiles; each starts at a different step of the
    // slice (and wraps) so that they do not all pull the same L2 lines at the same time
    const int rot = n_steps > 0 ? (unit * 5) % n_steps : 0;
    int fetch = step0 + rot;                   // next step to fetch
    auto fetch_next = [&](int slot_) {
        issue(fetch, slot_);
        fetch = fetch + 1 == step1 ? step0 : fetch + 1;
    };
    if constexpr (PRODUCER) {
        if (wave8 == 8) {
            // ---- the DMA wave: 5 + TILES instructions a stage (four pieces of nibbles, the scales, one per 16 rows of A) ----
            constexpr int PER = 5 + TILES;
            __builtin_amdgcn_s_setprio(3);      // its few instructions first: the others wait for what it requests (3 % of a launch)
            uint32_t a_voff[TILES];
#pragma unroll
            for (int t = 0; t < TILES; ++t)
                a_voff[t] = (uint32_t)((long)min(m0 + 16 * t + (lane >> 2), p.M - 1) * p.lda * 2 + 16 * a_chunk);
            auto issue_all = [&](int slot_) {
                uint8_t *st = lds + slot_ * GS_BYTES;
                const uint8_t *tile = w_base + (long)fetch * TILE_BYTES;
                const uint8_t *arow = a_base + (long)fetch * 64;
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    __builtin_amdgcn_global_load_lds((gptr_t)(tile + q * 1024 + lane * 16), (lptr_t)(st + q * 1024), 16, 0, 0);
                __builtin_amdgcn_global_load_lds((gptr_t)(tile + TILE_W_BYTES + lane * 4), (lptr_t)(st + GS_W), 4, 0, 0);
#pragma unroll
                for (int t = 0; t < TILES; ++t)
                    __builtin_amdgcn_global_load_lds((gptr_t)(arow + a_voff[t]), (lptr_t)(st + GS_W + GS_S + t * 1024), 16, 0, 0);
                fetch = fetch + 1 == step1 ? step0 : fetch + 1;
            };
#pragma unroll
            for (int i = 0; i < SLOTS - 2; ++i)
                if (i < n_steps) issue_all(i);
            if (n_steps > 0) {
                gemm_wait_dma<PER>(min(SLOTS - 3, n_steps - 1));
                gemm_barrier();
                int slot = 0;
                auto back = [&](int k) { return slot >= k ? slot - k : slot + SLOTS - k; };
                int i = 0;
#pragma unroll 1
                for (; i + SLOTS - 1 < n_steps; i += 2) {
                    gemm_wait_vm<PER * (SLOTS - 5)>();
                    gemm_barrier();
                    issue_all(back(2));
                    issue_all(back(1));
                    slot = slot + 2 >= SLOTS ? slot + 2 - SLOTS : slot + 2;
                }
#pragma unroll 1
                for (; i < n_steps; i += 2) {
                    gemm_wait_dma<PER>(max(0, min(n_steps - 1, i + SLOTS - 3) - (i + 2)));      // stages issued past step i + 2
                    gemm_barrier();
                    if (i + SLOTS - 2 < n_steps) issue_all(back(2));
                    if (i + SLOTS - 1 < n_steps) issue_all(back(1));
                    slot = slot + 2 >= SLOTS ? slot + 2 - SLOTS : slot + 2;
                }
            }
            // the barriers of the epilogue: one that frees the ring, one per row tile
#pragma unroll 1
            for (int t = 0; t < 1 + TILES + (more ? 1 : 0); ++t) gemm_barrier();
            return;
        }
    } else {
#pragma unroll
        for (int i = 0; i < SLOTS - 2; ++i)
            if (i < n_steps) fetch_next(i);
    }

    // the eight dwords of this lane's column bytes and of their scales, for one step
    auto load_ws = [&](const uint8_t *st, uint32_t (&wv)[8], uint32_t (&sv)[8]) {
        if (TILED) {
            // wv[0..3] = (x, x2) of byte 2bp, (x, x2) of byte 2bp+1; sv[0..3] / sv[4..7] = the row pairs' scales of the
            // block's first / second 64 columns
            const u32x4 wq = *reinterpret_cast<const u32x4 *>(st + wave * 1024 + lane * 16);
            if (WAVES == 8) {                  // the scales of this wave's nibble only
                const u32x4 sc = *reinterpret_cast<const u32x4 *>(st + GS_W + g * 64 + (2 * blk + hh) * 16);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    wv[r] = wq[r];
                    wv[4 + r] = 0;
                    sv[r] = sc[r];
                    sv[4 + r] = 0;
                }
                return;
            }
            const u32x4 sh = *reinterpret_cast<const u32x4 *>(st + GS_W + g * 64 + (2 * blk) * 16);
            const u32x4 sl = *reinterpret_cast<const u32x4 *>(st + GS_W + g * 64 + (2 * blk + 1) * 16);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                wv[r] = wq[r];
                wv[4 + r] = 0;
                sv[r] = sh[r];
                sv[4 + r] = sl[r];
            }
            return;
        }
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            wv[r] = *reinterpret_cast<const uint32_t *>(st + g * GS_WBLOCK + r * 128 + 64 * blk + 4 * c);
            sv[r] = *reinterpret_cast<const uint32_t *>(st + GS_W + (8 * g + r) * 8 + 4 * blk);
        }
    };
    // exact fp16 code * scale, as the four B operands (byte 2bp high / low, byte 2bp+1 high / low)
    // eight waves: the nibble this wave decodes, as constants of one and-or + one packed fma (code = fp16 bits * mul + off)
    const uint32_t nib_mask = hh == 0 ? 0x00F000F0u : 0x000F000Fu;
    uint32_t nib_magic = MAGIC_1024;                             // in a register the compiler cannot see through: (bits & mask) | magic is
    asm volatile("" : "+v"(nib_magic));                       // then ONE v_and_or_b32 (no literal operands there), not an AND and an OR
    const h2 nib_mul = hh == 0 ? h2{(half_t)0.0625f, (half_t)0.0625f} : h2{(half_t)1.0f, (half_t)1.0f};
    const h2 nib_off = hh == 0 ? h2{(half_t)-72.0f, (half_t)-72.0f} : h2{(half_t)-1032.0f, (half_t)-1032.0f};
    auto decode = [&](const uint32_t (&wv)[8], const uint32_t (&sv)[8], bool dead, h8 (&b)[NB]) {
        u32x4 v0h, v0l, v1h, v1l;
        if (TILED && WAVES == 8) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t pr0 = j < 2 ? wv[j] : wv[j - 2] >> 8;           // rows (2j, 2j+1) of byte 2bp, codes + 8
                const uint32_t pr1 = j < 2 ? wv[2 + j] : wv[j] >> 8;           // ... of byte 2bp+1
                const h2 sc = as_h2(sv[j]);
                v0h[j] = as_u32(__builtin_elementwise_fma(as_h2((pr0 & nib_mask) | nib_magic), nib_mul, nib_off) * sc);
                v1h[j] = as_u32(__builtin_elementwise_fma(as_h2((pr1 & nib_mask) | nib_magic), nib_mul, nib_off) * sc);
            }
            b[0] = __builtin_bit_cast(h8, v0h);
            b[1] = __builtin_bit_cast(h8, v1h);
            return;
        }
        if (TILED) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t pr0 = j < 2 ? wv[j] : wv[j - 2] >> 8;           // rows (2j, 2j+1) of byte 2bp, codes + 8
                const uint32_t pr1 = j < 2 ? wv[2 + j] : wv[j] >> 8;           // ... of byte 2bp+1
                const h2 s_hi = as_h2(sv[j]), s_lo = as_h2(sv[4 + j]);
                v0h[j] = as_u32(codes_high(pr0) * s_hi);
                v0l[j] = as_u32(codes_low(pr0) * s_lo);
                v1h[j] = as_u32(codes_high(pr1) * s_hi);
                v1l[j] = as_u32(codes_low(pr1) * s_lo);
            }
            if constexpr (NB == 4) {
                b[0] = __builtin_bit_cast(h8, v0h);
                b[1] = __builtin_bit_cast(h8, v0l);
                b[2] = __builtin_bit_cast(h8, v1h);
                b[3] = __builtin_bit_cast(h8, v1l);
            }
            return;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t pr0 = __builtin_amdgcn_perm(wv[2 * j + 1], wv[2 * j], sel0) ^ 0x00880088u;
            const uint32_t pr1 = __builtin_amdgcn_perm(wv[2 * j + 1], wv[2 * j], sel1) ^ 0x00880088u;
            const h2 s_hi = as_h2(pack_lo16(sv[2 * j], sv[2 * j + 1]));
            const h2 s_lo = as_h2(pack_hi16(sv[2 * j], sv[2 * j + 1]));
            v0h[j] = as_u32(codes_high(pr0) * s_hi);
            v0l[j] = as_u32(codes_low(pr0) * s_lo);
            v1h[j] = as_u32(codes_high(pr1) * s_hi);
            v1l[j] = as_u32(codes_low(pr1) * s_lo);
        }
        if (RAGGED && dead) v0h = v0l = v1h = v1l = u32x4{0u, 0u, 0u, 0u};     // k >= K: no contribution
        if constexpr (NB == 4) {
            b[0] = __builtin_bit_cast(h8, v0h);
            b[1] = __builtin_bit_cast(h8, v0l);
            b[2] = __builtin_bit_cast(h8, v1h);
            b[3] = __builtin_bit_cast(h8, v1l);
        }
    };
    auto k_dead = [&](int step) { return step * 32 + 8 * g >= p.K; };      // only in the last step when K % 32 != 0
    // While the matrix pipe multiplies step i (A tile read from stage i, B operands decoded one iteration
    // earlier), the wave reads the nibbles of step i+1 from LDS and decodes them.  After the barrier of
    // iteration i every wave has finished iteration i-1, so the slot of stage i-1 is refilled with step i+5.
    auto load_a = [&](const uint8_t *st, h8 (&av)[TILES]) {
        const uint8_t *at = st + GS_W + GS_S;
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
            const int r = 16 * t + c;
            av[t] = *reinterpret_cast<const h8 *>(at + r * 64 + ((g ^ ((r >> 2) & 3)) << 4));
        }
    };
    auto multiply = [&](const h8 (&av)[TILES], const h8 (&b)[NB]) {
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
#pragma unroll
            for (int o = 0; o < NB; ++o) acc[o][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[t], b[o], acc[o][t], 0, 0, 0);
        }
    };
    // Steps go in pairs: ONE wait + barrier per two steps.  With S slots (six; more only with the DMA wave): at the barrier
    // before steps i, i+1 the stages of steps i .. i+2 have landed (the B operands of step i+2 are decoded during step i+1),
    // steps i+3 .. i+S-3 may be in flight, and the slots of steps i-2, i-1 are refilled with steps i+S-2, i+S-1.  A stage has the same two steps of time to land as
    // with a barrier per step; the waves meet half as often.
    if (n_steps > 0) {
        h8 bq[NB];
        int cur = step0 + rot;                 // step being multiplied
        int slot = 0;                          // its ring slot
        {
            if constexpr (!PRODUCER) gemm_wait_dma<DMA_PER>(min(SLOTS - 3, n_steps - 1));
            gemm_barrier();
            uint32_t wv[8], sv[8];
            load_ws(lds, wv, sv);
            decode(wv, sv, k_dead(cur), bq);
        }
        // multiply the step in `slot` with bq while the B operands of the next step are decoded
        auto one_step = [&]() {
            const uint8_t *st = lds + slot * GS_BYTES;
            slot = slot == SLOTS - 1 ? 0 : slot + 1;
            cur = cur + 1 == step1 ? step0 : cur + 1;
            // past the last step the next slot holds stale bytes: read, decoded and never used
            uint32_t wv[8], sv[8];
            h8 av[TILES], bn[NB];
            load_a(st, av);
            load_ws(lds + slot * GS_BYTES, wv, sv);
            multiply(av, bq);
            decode(wv, sv, k_dead(cur), bn);
#pragma unroll
            for (int o = 0; o < NB; ++o) bq[o] = bn[o];
        };
        auto back = [&](int k) { return slot >= k ? slot - k : slot + SLOTS - k; };
        int i = 0;
#pragma unroll 1
        for (; i + SLOTS - 1 < n_steps; i += 2) {      // both refills exist: the body is one basic block
            if constexpr (!PRODUCER) gemm_wait_vm<DMA_PER * (SLOTS - 5)>();
            gemm_barrier();
            if constexpr (PRODUCER) {
                one_step();
                one_step();
            } else if constexpr (TILED && WAVES == 8 && TILES < 8) {       // (with all 8 row tiles, the prefill, this form measured 5-8 % slower)
                // the nibbles and scales of the two refills now, their A rows from inside the steps: the address unit takes
                // 16 cycles per instruction, and between MFMAs the wave has them to spare (2 % off a launch at 100 rows;
                // the nibbles and scales too from inside the steps, behind their branches: 4 % slower)
                const int sa = back(2), sb = back(1);
                const int fa = fetch, fb = fetch + 1 == step1 ? step0 : fetch + 1;
                fetch = fb + 1 == step1 ? step0 : fb + 1;
                issue_ws8(fa, sa);
                issue_ws8(fb, sb);
                for (int half = 0; half < 2; ++half) {
                    const uint8_t *st = lds + slot * GS_BYTES;
                    slot = slot == SLOTS - 1 ? 0 : slot + 1;
                    cur = cur + 1 == step1 ? step0 : cur + 1;
                    uint32_t wv[8], sv[8];
                    h8 av[TILES], bn[NB];
                    load_a(st, av);
                    load_ws(lds + slot * GS_BYTES, wv, sv);
                    constexpr int T0 = TILES / 2;
#pragma unroll
                    for (int t = 0; t < T0; ++t)
#pragma unroll
                        for (int o = 0; o < NB; ++o) acc[o][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[t], bq[o], acc[o][t], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                    issue_a8(half == 0 ? fa : fb, half == 0 ? sa : sb);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int t = T0; t < TILES; ++t)
#pragma unroll
                        for (int o = 0; o < NB; ++o) acc[o][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[t], bq[o], acc[o][t], 0, 0, 0);
                    decode(wv, sv, k_dead(cur), bn);
#pragma unroll
                    for (int o = 0; o < NB; ++o) bq[o] = bn[o];
                }
            } else {
                fetch_next(back(2));
                fetch_next(back(1));
                one_step();
                one_step();
            }
        }
#pragma unroll 1
        for (; i < n_steps; i += 2) {
            if constexpr (!PRODUCER) gemm_wait_dma<DMA_PER>(max(0, min(n_steps - 1, i + SLOTS - 3) - (i + 2)));      // stages issued past step i + 2
            gemm_barrier();
            if constexpr (!PRODUCER) {
                if (i + SLOTS - 2 < n_steps) fetch_next(back(2));
                if (i + SLOTS - 1 < n_steps) fetch_next(back(1));
            }
            one_step();
            if (i + 1 < n_steps) one_step();
        }
    }

    // ---- results leave one 16-row tile at a time through LDS: [16][256 + 4] floats, two buffers in turn ----
    // accumulator element r of acc[o][t] is row 16t + 4g + r, column 128*blk + 64*(o&1) + 4c + 2*bp + (o>>1).
    // Bare barriers again: __syncthreads() would wait for the global stores of the previous tile to be
    // acknowledged, one memory round trip per tile.  A buffer is rewritten two tiles later, after a barrier
    // that every wave reaches only when its reads of that buffer have returned.
    constexpr int OP = GEMM_COLS + 4;
    constexpr int OTILE_BYTES = 16 * OP * 4;
    static_assert(2 * OTILE_BYTES <= SLOTS * GS_BYTES, "two output tiles must fit in the ring");
    float *slab = p.partial + (long)slice * p.M * p.n_total;
    const int o_row = (tid & 255) >> 4;         // 0..15
    const int o_half = tid >> 8;                // eight waves: the second 256 threads store the second half of the columns
    const int o_lane = tid & 15;                // store q of this lane: columns 64q + 4*o_lane .. (fp16: 128q + 8*o_lane ..),
                                                // so that one store instruction writes whole contiguous rows
    gemm_barrier();                             // every wave has left the main loop: the ring is free
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
        float *otile = reinterpret_cast<float *>(lds + (t & 1) * OTILE_BYTES);
        // operands o and o + 2 are neighbouring columns: one 8-byte LDS store for the pair
        if constexpr (WAVES == 8) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                *reinterpret_cast<f2 *>(&otile[(4 * g + r) * OP + 128 * blk + 64 * hh + 4 * c + 2 * bp]) = f2{acc[0][t][r], acc[1][t][r]};
        } else {
#pragma unroll
            for (int o = 0; o < 2; ++o)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    *reinterpret_cast<f2 *>(&otile[(4 * g + r) * OP + 128 * blk + 64 * o + 4 * c + 2 * bp]) = f2{acc[o][t][r], acc[o + 2][t][r]};
        }
        gemm_barrier();
        const int m = m0 + 16 * t + o_row;
        if (m < p.M) {
            if (p.direct) {
#pragma unroll
                for (int q = (WAVES == 8 ? o_half : 0); q < (WAVES == 8 ? o_half + 1 : 2); ++q) {
                    const int n_seg = col0 + 128 * q + 8 * o_lane;
                    if (n_seg < seg.N) {
                        const int n = seg.col0 + n_seg;
                        const f4 v0 = *reinterpret_cast<const f4 *>(otile + o_row * OP + 128 * q + 8 * o_lane);
                        const f4 v1 = *reinterpret_cast<const f4 *>(otile + o_row * OP + 128 * q + 8 * o_lane + 4);
                        h8 o;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            o[e] = matmul_epilogue(p, v0[e], m, n + e);
                            o[4 + e] = matmul_epilogue(p, v1[e], m, n + 4 + e);
                        }
                        *reinterpret_cast<h8 *>(p.c + (long)m * p.ldc + n) = o;
                    }
                }
            } else {
                float *dst = slab + (long)m * p.n_total + seg.col0 + col0;
#pragma unroll
                for (int q = (WAVES == 8 ? 2 * o_half : 0); q < (WAVES == 8 ? 2 * o_half + 2 : 4); ++q) {
                    const int cq = 64 * q + 4 * o_lane;
                    if (col0 + cq < seg.N) *reinterpret_cast<f4 *>(dst + cq) = *reinterpret_cast<const f4 *>(otile + o_row * OP + cq);
                }
            }
        }
    }
    if (zero_rest) {
        for (int sl = slice + 1; sl < p.ksplit; ++sl) {
            float *zslab = p.partial + (long)sl * p.M * p.n_total;
            for (int t = 0; t < TILES; ++t) {
                const int m = m0 + 16 * t + o_row;
                if (m < p.M) {
                    float *dst = zslab + (long)m * p.n_total + seg.col0 + col0;
#pragma unroll
                    for (int q = (WAVES == 8 ? 2 * o_half : 0); q < (WAVES == 8 ? 2 * o_half + 2 : 4); ++q) {
                        const int cq = 64 * q + 4 * o_lane;
                        if (col0 + cq < seg.N) *reinterpret_cast<f4 *>(dst + cq) = f4{0.f, 0.f, 0.f, 0.f};
                    }
                }
            }
        }
    }
    if (more) gemm_barrier();                   // the next piece refills the ring the last row tile left through
}

// PRODUCER (eight waves only): a ninth wave issues every DMA instruction of the workgroup and waits for them; the eight
// others only meet it at the barriers.  The compute unit's address unit takes 16 cycles per DMA instruction, during which
// the issuing wave stands still: ~0.28 us per pair of steps off the multiplying waves' path.  For launches with one
// workgroup per compute unit (a ninth and tenth wave on a SIMD that already holds four would cap the registers below
// what the kernel needs).  SLOTS: slots of the ring.
// RANGE (p.chunk > 0): the steps of all column units, laid end to end, are dealt in runs of p.chunk to the workgroups, one
// workgroup per compute unit, so a workgroup may finish one unit and begin the next: up to two pieces, one after the other.
template <int TILES, bool RAGGED, bool TILED, int WAVES, int SLOTS = GEMM_STAGES, bool PRODUCER = false, bool RANGE = false>
__global__ __launch_bounds__(64 * (WAVES + (PRODUCER ? 1 : 0)), WAVES == 8 ? 1 : 2) void q40_gemm_kernel(MatmulParams p) {
    static_assert(WAVES == 4 || (WAVES == 8 && TILED && !RAGGED), "eight waves: tiled weights, K a multiple of 32");
    static_assert(SLOTS >= 6 && SLOTS <= 10 && (SLOTS == GEMM_STAGES || PRODUCER) && (!PRODUCER || WAVES == 8), "ring depth");
    const int steps_total = (p.K + 31) / 32;
    if constexpr (RANGE) {
        int run0 = (int)blockIdx.x * p.chunk;                  // (units x steps is far below 2^31)
        const int run1 = min(run0 + p.chunk, p.units * steps_total);
#pragma unroll 1
        for (bool more = true; more;) {                        // (a loop, not two calls: the second piece runs code that is warm)
            const int unit = run0 / steps_total;
            const int s0 = run0 - unit * steps_total;
            const int s1 = min(steps_total, s0 + (run1 - run0));
            const int first = (unit * steps_total) / p.chunk;  // the workgroup that holds the unit's first piece
            run0 += s1 - s0;
            more = run0 < run1;
            // a zero the compiler cannot see keeps everything derived from the thread index inside the piece: hoisted out of
            // this loop those values stay live through it and the kernel spills
            int opaque_zero;
            asm volatile("s_mov_b32 %0, 0" : "=s"(opaque_zero));
            gemm_piece<TILES, RAGGED, TILED, WAVES, SLOTS, PRODUCER>(p, unit, 0, (int)blockIdx.x - first, s0, s1, s1 == steps_total, more, opaque_zero);
        }
    } else {
        int bid = blockIdx.x;
        // slot -> unit: each XCD (blockIdx % 8) takes a contiguous run of column units, which share scale lines
        const int slot = bid % p.units_pad;  bid /= p.units_pad;
        const int unit = (slot & 7) * (p.units_pad >> 3) + (slot >> 3);
        if (unit >= p.units) return;
        const int mb = bid % p.mblocks;
        const int slice = bid / p.mblocks;
        const int s0 = slice * p.steps_per_slice;
        gemm_piece<TILES, RAGGED, TILED, WAVES, SLOTS, PRODUCER>(p, unit, mb, slice, s0, min(s0 + p.steps_per_slice, steps_total), false, false, 0);
    }
}

// ---- two K-groups in one workgroup (tiled weights, K a multiple of 64, one workgroup per compute unit) ----------------
// A workgroup owns ONE 128-column block (pieces 2 blk, 2 blk + 1 of the unit's tiles), a block of rows and a K-slice, and
// its eight multiplying waves form two groups: group kk takes the steps 2 i + kk of the slice.  Wave (kk, hh, bp)
// multiplies the columns of nibble hh of piece 2 blk + bp of its group's steps with all row tiles of A - the same two B
// operands and 14 MFMAs per step as in q40_gemm_kernel - so a ring stage holds TWO steps: both pieces of the block and the
// scales of either step, and either step's rows of A.  The groups' accumulators are added through LDS at the end (group 0
// + group 1, a fixed order), and all eight waves write the slab.  Against q40_gemm_kernel's 256-column units this
// fills the GPU with half as many K-slices, i.e. half the slab bytes written here and read back by the consumer; the
// price is that a row of A is staged for 128 columns instead of 256.
constexpr int KG_W = 4096;                     // [group kk][piece bp] x 1024
constexpr int KG_S = 512;                      // [group kk] x 256 (the whole scale block of the step)
template <int TILES> struct KgShape {
    static constexpr int STAGE = KG_W + KG_S + 2 * TILES * 1024;
    static constexpr int SLOTS = GEMM_DMA_WAVE_SLOTS;
    static constexpr int RING = SLOTS * STAGE;
    static constexpr int PER = 2 * (3 + TILES);                    // DMA instructions of a stage
    static constexpr int OP = 128 + 4;                             // floats per row of a group's sums in LDS
    static constexpr int SUMS = TILES * 16 * OP * 4;               // one K-group's sums: [row][OP] fp32
    static constexpr int LDS = RING > 2 * SUMS ? RING : 2 * SUMS;
    static_assert(PER * (SLOTS - 5) <= 63 && LDS <= 160 * 1024, "ring");
};

template <int TILES>
__global__ __launch_bounds__(576, 1) void q40_gemm_kg_kernel(MatmulParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    typedef KgShape<TILES> S;
    constexpr int SLOTS = S::SLOTS, PER = S::PER, STAGE = S::STAGE;
    const int tid = threadIdx.x;
    const int wave8 = __builtin_amdgcn_readfirstlane(tid >> 6);       // 0..7 multiply, 8 issues the DMA
    const int lane = tid & 63, c = lane & 15, g = lane >> 4;
    // blockIdx -> (128-column block, row block, K-slice); blocks of one unit are neighbours (same XCD every 8)
    int bid = blockIdx.x;
    const int hb = bid % (2 * p.units_pad);  bid /= 2 * p.units_pad;
    const int slot_u = hb >> 1, blk = hb & 1;
    const int unit = (slot_u & 7) * (p.units_pad >> 3) + (slot_u >> 3);
    if (unit >= p.units) return;
    const int mb = bid % p.mblocks, slice = bid / p.mblocks;
    int sg = 0;
    if (p.nseg > 1 && unit >= p.seg[1].unit0) sg = 1;
    if (p.nseg > 2 && unit >= p.seg[2].unit0) sg = 2;
    const MatmulSegment seg = p.seg[sg];
    const int pair = unit - seg.unit0;
    const int col0 = pair * GEMM_COLS + 128 * blk;
    if (col0 >= seg.N) return;                                         // a weight with an odd number of 128-column blocks
    const int m0 = mb * p.block_rows;
    const int steps_total = p.K / 32;
    const int step0 = slice * p.steps_per_slice, step1 = min(step0 + p.steps_per_slice, steps_total);
    const int n_st = max(step1 - step0, 0) / 2;                        // stages (two steps each; slices are even)
    const uint8_t *w_base = seg.w + (long)pair * tiled_steps(p.K) * TILE_BYTES + (long)step0 * TILE_BYTES;
    const uint8_t *a_base = reinterpret_cast<const uint8_t *>(p.a) + (long)step0 * 64;
    const int rot = n_st > 0 ? (hb * 5) % n_st : 0;                   // workgroups of a K-slice start at different stages

    if (wave8 == 8) {
        // ---- the DMA wave ----
        __builtin_amdgcn_s_setprio(3);
        const int a_chunk = (lane & 3) ^ ((lane >> 4) & 3);
        uint32_t a_voff[TILES];
#pragma unroll
        for (int t = 0; t < TILES; ++t)
            a_voff[t] = (uint32_t)((long)min(m0 + 16 * t + (lane >> 2), p.M - 1) * p.lda * 2 + 16 * a_chunk);
        int fetch = rot;
        auto issue_stage = [&](int slot_) {
            uint8_t *st = lds + slot_ * STAGE;
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
                const uint8_t *tile = w_base + (long)(2 * fetch + kk) * TILE_BYTES;
                const uint8_t *arow = a_base + (long)(2 * fetch + kk) * 64;
#pragma unroll
                for (int bp = 0; bp < 2; ++bp)
                    __builtin_amdgcn_global_load_lds((gptr_t)(tile + (2 * blk + bp) * 1024 + lane * 16), (lptr_t)(st + (2 * kk + bp) * 1024), 16, 0, 0);
                __builtin_amdgcn_global_load_lds((gptr_t)(tile + TILE_W_BYTES + lane * 4), (lptr_t)(st + KG_W + kk * 256), 4, 0, 0);
#pragma unroll
                for (int t = 0; t < TILES; ++t)
                    __builtin_amdgcn_global_load_lds((gptr_t)(arow + a_voff[t]), (lptr_t)(st + KG_W + KG_S + (kk * TILES + t) * 1024), 16, 0, 0);
            }
            fetch = fetch + 1 == n_st ? 0 : fetch + 1;
        };
#pragma unroll
        for (int i = 0; i < SLOTS - 2; ++i)
            if (i < n_st) issue_stage(i);
        if (n_st > 0) {
            gemm_wait_dma<PER>(min(SLOTS - 3, n_st - 1));
            gemm_barrier();
            int slot = 0;
            auto back = [&](int k) { return slot >= k ? slot - k : slot + SLOTS - k; };
            int i = 0;
#pragma unroll 1
            for (; i + SLOTS - 1 < n_st; i += 2) {
                gemm_wait_vm<PER * (SLOTS - 5)>();
                gemm_barrier();
                issue_stage(back(2));
                issue_stage(back(1));
                slot = slot + 2 >= SLOTS ? slot + 2 - SLOTS : slot + 2;
            }
#pragma unroll 1
            for (; i < n_st; i += 2) {
                gemm_wait_dma<PER>(max(0, min(n_st - 1, i + SLOTS - 3) - (i + 2)));
                gemm_barrier();
                if (i + SLOTS - 2 < n_st) issue_stage(back(2));
                if (i + SLOTS - 1 < n_st) issue_stage(back(1));
                slot = slot + 2 >= SLOTS ? slot + 2 - SLOTS : slot + 2;
            }
        }
        gemm_barrier();                                        // the epilogue's two barriers: ring free, sums in place
        gemm_barrier();
        return;
    }

    const int kk = wave8 >> 2, hh = (wave8 >> 1) & 1, bp = wave8 & 1;
    const uint32_t nib_mask = hh == 0 ? 0x00F000F0u : 0x000F000Fu;
    uint32_t nib_magic = MAGIC_1024;                             // in a register the compiler cannot see through: (bits & mask) | magic is
    asm volatile("" : "+v"(nib_magic));                       // then ONE v_and_or_b32 (no literal operands there), not an AND and an OR
    const h2 nib_mul = hh == 0 ? h2{(half_t)0.0625f, (half_t)0.0625f} : h2{(half_t)1.0f, (half_t)1.0f};
    const h2 nib_off = hh == 0 ? h2{(half_t)-72.0f, (half_t)-72.0f} : h2{(half_t)-1032.0f, (half_t)-1032.0f};
    struct Raw { u32x4 wq, sc; };
    auto load_ws = [&](const uint8_t *st, Raw &r) {
        r.wq = *reinterpret_cast<const u32x4 *>(st + (2 * kk + bp) * 1024 + lane * 16);
        r.sc = *reinterpret_cast<const u32x4 *>(st + KG_W + kk * 256 + g * 64 + (2 * blk + hh) * 16);
    };
    auto decode = [&](const Raw &r, h8 (&b)[2]) {
        u32x4 v0, v1;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t pr0 = j < 2 ? r.wq[j] : r.wq[j - 2] >> 8;       // rows (2j, 2j+1) of byte 2bp, codes + 8
            const uint32_t pr1 = j < 2 ? r.wq[2 + j] : r.wq[j] >> 8;       // ... of byte 2bp+1
            const h2 sc = as_h2(r.sc[j]);
            v0[j] = as_u32(__builtin_elementwise_fma(as_h2((pr0 & nib_mask) | nib_magic), nib_mul, nib_off) * sc);
            v1[j] = as_u32(__builtin_elementwise_fma(as_h2((pr1 & nib_mask) | nib_magic), nib_mul, nib_off) * sc);
        }
        b[0] = __builtin_bit_cast(h8, v0);
        b[1] = __builtin_bit_cast(h8, v1);
    };
    auto load_a = [&](const uint8_t *st, h8 (&av)[TILES]) {
        const uint8_t *at = st + KG_W + KG_S + kk * TILES * 1024;
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
            const int r = 16 * t + c;
            av[t] = *reinterpret_cast<const h8 *>(at + r * 64 + ((g ^ ((r >> 2) & 3)) << 4));
        }
    };
    f4 acc[2][TILES];
#pragma unroll
    for (int o = 0; o < 2; ++o)
#pragma unroll
        for (int t = 0; t < TILES; ++t) acc[o][t] = f4{0.f, 0.f, 0.f, 0.f};

    if (n_st > 0) {
        h8 bq[2];
        int slot = 0;
        gemm_barrier();
        {
            Raw r;
            load_ws(lds, r);
            decode(r, bq);
        }
        auto one_stage = [&]() {
            const uint8_t *st = lds + slot * STAGE;
            slot = slot == SLOTS - 1 ? 0 : slot + 1;
            Raw r;
            h8 av[TILES], bn[2];
            load_a(st, av);
            load_ws(lds + slot * STAGE, r);                    // (past the last stage: stale bytes, decoded and never used)
#pragma unroll
            for (int t = 0; t < TILES; ++t)
#pragma unroll
                for (int o = 0; o < 2; ++o) acc[o][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[t], bq[o], acc[o][t], 0, 0, 0);
            decode(r, bn);
            bq[0] = bn[0];
            bq[1] = bn[1];
        };
        int i = 0;
#pragma unroll 1
        for (; i + 1 < n_st; i += 2) {
            gemm_barrier();
            one_stage();
            one_stage();
        }
        if (i < n_st) {
            gemm_barrier();
            one_stage();
        }
    }

    // ---- both groups' sums as rows of 128 floats in LDS; then every thread adds group 0 + group 1 (a fixed order) for
    // 16-byte runs of whole rows and writes the slab: one pass, two barriers, all eight waves storing ----
    gemm_barrier();                                            // every wave has left the loop: the ring is free
    constexpr int OP = S::OP;
    {
        float *sums = reinterpret_cast<float *>(lds + kk * S::SUMS);
#pragma unroll
        for (int t = 0; t < TILES; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                *reinterpret_cast<f2 *>(&sums[(16 * t + 4 * g + r) * OP + 64 * hh + 4 * c + 2 * bp]) = f2{acc[0][t][r], acc[1][t][r]};
    }
    gemm_barrier();
    const float *sum0 = reinterpret_cast<const float *>(lds), *sum1 = reinterpret_cast<const float *>(lds + S::SUMS);
    float *slab = p.partial + (long)slice * p.M * p.n_total + seg.col0 + col0;
#pragma unroll
    for (int it = 0; it < TILES; ++it) {
        const int idx = tid + 512 * it;                        // tid < 512 here: (row, run of four columns)
        const int row = idx >> 5, cq = 4 * (idx & 31);
        const int m = m0 + row;
        if (m < p.M && row < p.block_rows) {
            const f4 v = *reinterpret_cast<const f4 *>(sum0 + row * OP + cq) + *reinterpret_cast<const f4 *>(sum1 + row * OP + cq);
            *reinterpret_cast<f4 *>(slab + (long)m * p.n_total + cq) = v;
        }
    }
}

// ---- SwiGLU inside the launch of w1|w3 (tiled weights, 17 .. 128 rows, all of K in one workgroup) -----------------------
// q40_gemm_kg_kernel with the roles of a workgroup's waves changed: instead of the two pieces of one 128-column block, a
// workgroup takes piece bp of block j of the GATE weight and the same piece of the UP weight (64 columns each, the same
// columns), so its wave (kk, hh, gu) holds, after the K-groups are added, gate or up for exactly the columns its neighbour
// holds the other for.  The epilogue forms fp16(silu(fp16(gate))) * fp16(up) with the roundings of partial_silu_mul_kernel
// and stores the activations of w2: no slab leaves the launch and the SiLU launch is gone.
template <int TILES> struct SwigluShape {
    static constexpr int SC = 1024;                                  // scales: [group kk][gate | up] x 256
    static constexpr int STAGE = KG_W + SC + 2 * TILES * 1024;
    static constexpr int SLOTS = GEMM_DMA_WAVE_SLOTS;
    static constexpr int LDS = SLOTS * STAGE;
    static constexpr int PER = 2 * (4 + TILES);
    static constexpr int RED = 4 * TILES * 2 * 1024;
    static constexpr int OP = 64 + 4;
    static constexpr int OTILE = 2 * 16 * OP * 4;
    static_assert(RED + 2 * OTILE <= LDS, "the sums of the second group and two output tiles must fit in the ring");
    static_assert(PER * (SLOTS - 5) <= 63 && LDS <= 160 * 1024, "ring");
};

template <int TILES>
__global__ __launch_bounds__(576, 1) void q40_gemm_swiglu_kernel(MatmulParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    typedef SwigluShape<TILES> S;
    constexpr int SLOTS = S::SLOTS, PER = S::PER, STAGE = S::STAGE;
    const int tid = threadIdx.x;
    const int wave8 = __builtin_amdgcn_readfirstlane(tid >> 6);       // 0..7 multiply, 8 issues the DMA
    const int lane = tid & 63, c = lane & 15, g = lane >> 4;
    // blockIdx -> (128-column block j of the gate and of the up weight, piece bp of that block)
    const int hb = blockIdx.x;
    const int blockj = hb >> 1, bp = hb & 1;
    const int pair = blockj >> 1, blk = blockj & 1;
    const int n_half = p.seg[0].N;
    if (128 * blockj >= n_half) return;
    constexpr int m0 = 0;
    const int n_st = p.K / 64;                                         // stages (two steps each), all of K
    const uint8_t *w_gate = p.seg[0].w + (long)pair * tiled_steps(p.K) * TILE_BYTES;
    const uint8_t *w_up = p.seg[1].w + (long)pair * tiled_steps(p.K) * TILE_BYTES;
    const uint8_t *a_base = reinterpret_cast<const uint8_t *>(p.a);
    const int rot = n_st > 0 ? (hb * 5) % n_st : 0;                   // workgroups of a K-slice start at different stages

    if (wave8 == 8) {
        // ---- the DMA wave ----
        __builtin_amdgcn_s_setprio(3);
        const int a_chunk = (lane & 3) ^ ((lane >> 4) & 3);
        uint32_t a_voff[TILES];
#pragma unroll
        for (int t = 0; t < TILES; ++t)
            a_voff[t] = (uint32_t)((long)min(m0 + 16 * t + (lane >> 2), p.M - 1) * p.lda * 2 + 16 * a_chunk);
        int fetch = rot;
        auto issue_stage = [&](int slot_) {
            uint8_t *st = lds + slot_ * STAGE;
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
                const long off = (long)(2 * fetch + kk) * TILE_BYTES;
                const uint8_t *arow = a_base + (long)(2 * fetch + kk) * 64;
#pragma unroll
                for (int gu = 0; gu < 2; ++gu) {
                    const uint8_t *tile = (gu == 0 ? w_gate : w_up) + off;
                    __builtin_amdgcn_global_load_lds((gptr_t)(tile + (2 * blk + bp) * 1024 + lane * 16), (lptr_t)(st + (2 * kk + gu) * 1024), 16, 0, 0);
                    __builtin_amdgcn_global_load_lds((gptr_t)(tile + TILE_W_BYTES + lane * 4), (lptr_t)(st + KG_W + (2 * kk + gu) * 256), 4, 0, 0);
                }
#pragma unroll
                for (int t = 0; t < TILES; ++t)
                    __builtin_amdgcn_global_load_lds((gptr_t)(arow + a_voff[t]), (lptr_t)(st + KG_W + S::SC + (kk * TILES + t) * 1024), 16, 0, 0);
            }
            fetch = fetch + 1 == n_st ? 0 : fetch + 1;
        };
#pragma unroll
        for (int i = 0; i < SLOTS - 2; ++i)
            if (i < n_st) issue_stage(i);
        if (n_st > 0) {
            gemm_wait_dma<PER>(min(SLOTS - 3, n_st - 1));
            gemm_barrier();
            int slot = 0;
            auto back = [&](int k) { return slot >= k ? slot - k : slot + SLOTS - k; };
            int i = 0;
#pragma unroll 1
            for (; i + SLOTS - 1 < n_st; i += 2) {
                gemm_wait_vm<PER * (SLOTS - 5)>();
                gemm_barrier();
                issue_stage(back(2));
                issue_stage(back(1));
                slot = slot + 2 >= SLOTS ? slot + 2 - SLOTS : slot + 2;
            }
#pragma unroll 1
            for (; i < n_st; i += 2) {
                gemm_wait_dma<PER>(max(0, min(n_st - 1, i + SLOTS - 3) - (i + 2)));
                gemm_barrier();
                if (i + SLOTS - 2 < n_st) issue_stage(back(2));
                if (i + SLOTS - 1 < n_st) issue_stage(back(1));
                slot = slot + 2 >= SLOTS ? slot + 2 - SLOTS : slot + 2;
            }
        }
        // the barriers of the epilogue: ring free, second group's sums in place, one per row tile
#pragma unroll 1
        for (int t = 0; t < 2 + TILES; ++t) gemm_barrier();
        return;
    }

    const int kk = wave8 >> 2, hh = (wave8 >> 1) & 1, gu = wave8 & 1;       // K-group, nibble, gate (0) or up (1)
    const uint32_t nib_mask = hh == 0 ? 0x00F000F0u : 0x000F000Fu;
    uint32_t nib_magic = MAGIC_1024;                             // in a register the compiler cannot see through: (bits & mask) | magic is
    asm volatile("" : "+v"(nib_magic));                       // then ONE v_and_or_b32 (no literal operands there), not an AND and an OR
    const h2 nib_mul = hh == 0 ? h2{(half_t)0.0625f, (half_t)0.0625f} : h2{(half_t)1.0f, (half_t)1.0f};
    const h2 nib_off = hh == 0 ? h2{(half_t)-72.0f, (half_t)-72.0f} : h2{(half_t)-1032.0f, (half_t)-1032.0f};
    struct Raw { u32x4 wq, sc; };
    auto load_ws = [&](const uint8_t *st, Raw &r) {
        r.wq = *reinterpret_cast<const u32x4 *>(st + (2 * kk + gu) * 1024 + lane * 16);
        r.sc = *reinterpret_cast<const u32x4 *>(st + KG_W + (2 * kk + gu) * 256 + g * 64 + (2 * blk + hh) * 16);
    };
    auto decode = [&](const Raw &r, h8 (&b)[2]) {
        u32x4 v0, v1;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t pr0 = j < 2 ? r.wq[j] : r.wq[j - 2] >> 8;       // rows (2j, 2j+1) of byte 2bp, codes + 8
            const uint32_t pr1 = j < 2 ? r.wq[2 + j] : r.wq[j] >> 8;       // ... of byte 2bp+1
            const h2 sc = as_h2(r.sc[j]);
            v0[j] = as_u32(__builtin_elementwise_fma(as_h2((pr0 & nib_mask) | nib_magic), nib_mul, nib_off) * sc);
            v1[j] = as_u32(__builtin_elementwise_fma(as_h2((pr1 & nib_mask) | nib_magic), nib_mul, nib_off) * sc);
        }
        b[0] = __builtin_bit_cast(h8, v0);
        b[1] = __builtin_bit_cast(h8, v1);
    };
    auto load_a = [&](const uint8_t *st, h8 (&av)[TILES]) {
        const uint8_t *at = st + KG_W + S::SC + kk * TILES * 1024;
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
            const int r = 16 * t + c;
            av[t] = *reinterpret_cast<const h8 *>(at + r * 64 + ((g ^ ((r >> 2) & 3)) << 4));
        }
    };
    f4 acc[2][TILES];
#pragma unroll
    for (int o = 0; o < 2; ++o)
#pragma unroll
        for (int t = 0; t < TILES; ++t) acc[o][t] = f4{0.f, 0.f, 0.f, 0.f};

    if (n_st > 0) {
        h8 bq[2];
        int slot = 0;
        gemm_barrier();
        {
            Raw r;
            load_ws(lds, r);
            decode(r, bq);
        }
        auto one_stage = [&]() {
            const uint8_t *st = lds + slot * STAGE;
            slot = slot == SLOTS - 1 ? 0 : slot + 1;
            Raw r;
            h8 av[TILES], bn[2];
            load_a(st, av);
            load_ws(lds + slot * STAGE, r);                    // (past the last stage: stale bytes, decoded and never used)
#pragma unroll
            for (int t = 0; t < TILES; ++t)
#pragma unroll
                for (int o = 0; o < 2; ++o) acc[o][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[t], bq[o], acc[o][t], 0, 0, 0);
            decode(r, bn);
            bq[0] = bn[0];
            bq[1] = bn[1];
        };
        int i = 0;
#pragma unroll 1
        for (; i + 1 < n_st; i += 2) {
            gemm_barrier();
            one_stage();
            one_stage();
        }
        if (i < n_st) {
            gemm_barrier();
            one_stage();
        }
    }

    // ---- group 0 + group 1 through LDS, then the slab one row tile at a time ----
    gemm_barrier();                                            // every wave has left the loop: the ring is free
    if (kk == 1) {
        uint8_t *dst = lds + (wave8 - 4) * (TILES * 2 * 1024) + lane * 16;
#pragma unroll
        for (int t = 0; t < TILES; ++t)
#pragma unroll
            for (int o = 0; o < 2; ++o) *reinterpret_cast<f4 *>(dst + (t * 2 + o) * 1024) = acc[o][t];
    }
    gemm_barrier();
    if (kk == 1) {
#pragma unroll 1
        for (int t = 0; t < TILES; ++t) gemm_barrier();
        return;
    }
    {
        const uint8_t *src = lds + wave8 * (TILES * 2 * 1024) + lane * 16;
#pragma unroll
        for (int t = 0; t < TILES; ++t)
#pragma unroll
            for (int o = 0; o < 2; ++o) acc[o][t] += *reinterpret_cast<const f4 *>(src + (t * 2 + o) * 1024);
    }
    // rows of 64 columns: local column 32 hh + 2 c + o is column 128 blockj + 64 hh + 4 c + 2 bp + o of the weights
    constexpr int OP = S::OP;
    const int o_row = tid >> 4, o_lane = tid & 15;            // tid < 256 here
    const int st_hh = o_lane >> 3, st_c = 2 * (o_lane & 7);   // this thread's four local columns 4 o_lane .. + 3 when storing
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
        float *otile = reinterpret_cast<float *>(lds + S::RED + (t & 1) * S::OTILE);      // [gate | up][16][OP]
#pragma unroll
        for (int r = 0; r < 4; ++r)
            *reinterpret_cast<f2 *>(&otile[gu * 16 * OP + (4 * g + r) * OP + 32 * hh + 2 * c]) = f2{acc[0][t][r], acc[1][t][r]};
        gemm_barrier();
        const int m = 16 * t + o_row;
        if (m < p.M) {
            const f4 gv = *reinterpret_cast<const f4 *>(otile + o_row * OP + 4 * o_lane);
            const f4 uv = *reinterpret_cast<const f4 *>(otile + 16 * OP + o_row * OP + 4 * o_lane);
            half_t ov[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {                      // the roundings of partial_silu_mul_kernel
                const float gf = (float)(half_t)gv[e];
                const half_t sl = (half_t)(gf / (1.0f + expf(-gf)));
                ov[e] = sl * (half_t)uv[e];
            }
            half_t *dst = p.c + (long)m * p.ldc + 128 * blockj + 64 * st_hh + 4 * st_c + 2 * bp;
            *reinterpret_cast<h2 *>(dst) = h2{ov[0], ov[1]};
            *reinterpret_cast<h2 *>(dst + 4) = h2{ov[2], ov[3]};
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
    p.block_rows = GEMM_BM;
    p.kgroups = 0;
    // Tiled weights, 17 .. 128 rows, K a multiple of 64: 128-column blocks with two K-groups a workgroup (q40_gemm_kg_kernel)
    // where they fill at least two thirds of the compute units in one round - half the K-slices, or fewer, of the 256-column
    // units below for the same number of workgroups.  Narrow matrices (at most 32 blocks: wo, w2) at any such row count, and
    // with two 64-row blocks per column block where K is short (wo at 65 .. 128 rows); wide ones (wq|wk|wv, w1|w3) above
    // 64 rows only (below, the launch loses more than its consumer gains); K up to 16384 (a row of A is staged for 128 columns
    // instead of 256, which makes the loop ~12 % slower per step: with K = 28672 that outweighs the slabs).  Measured at 100
    // rows, launch + consumer: wo 15.8 against 17.5 us, w2 24.7 against 26.9, w1|w3 39.7 against 40.9; a decode step at 100
    // branches 4.06 against 4.29 ms.
    if (p.tiled && p.M <= 128 && p.K % 64 == 0 && p.K <= 16384) {
        int blocks = 0;
        for (int i = 0; i < p.nseg; ++i) blocks += p.seg[i].N / 128;
        const bool narrow = blocks <= 32;
        const int mblocks = (narrow && p.M > 64 && p.K <= 4096) ? 2 : 1;
        int ks = 256 / (blocks * mblocks);
        int cap = GEMM_KSCAP / p.M;
        if (cap > SMH_MAX_KSPLIT) cap = SMH_MAX_KSPLIT;
        if (ks > cap) ks = cap;
        const int steps = p.K / 32;
        if (ks > steps / 8) ks = steps / 8;                    // at least four stages (of two steps) a slice
        if (ks >= 1 && (narrow || p.M > 64) && (long)blocks * mblocks * ks >= 170) {
            p.kgroups = 2;
            p.mblocks = mblocks;
            p.block_rows = mblocks == 2 ? 64 : GEMM_BM;
            p.chunk = 0;
            int sps = (steps + ks - 1) / ks;
            sps += sps & 1;                                    // a stage of the ring is two steps
            p.steps_per_slice = sps;
            p.ksplit = (steps + sps - 1) / sps;
            return;
        }
    }
    // 65 .. 128 rows of a matrix with few column units and a short K (wo at 100 branches): two 64-row blocks per unit take
    // half as many K-slices to fill the GPU, so half the slab bytes are written here and read by the consumer.  The blocks
    // of a unit read the same weights at the same time in the same XCD.  (Measured at 100 rows: wo and the RMSNorm behind
    // it 17.1 us against 19.8; with K = 11008 the launch itself loses what the consumer gains, 43 steps a workgroup.)
    if (p.M > 64 && p.M <= 128 && p.units <= 16 && p.K % 32 == 0 && p.K <= 4096) p.block_rows = 64;
    p.mblocks = (p.M + p.block_rows - 1) / p.block_rows;
    const int steps = (p.K + 31) / 32;
    const long tiles = (long)p.units * p.mblocks;
    // One round of workgroups.  One workgroup per compute unit when the column units divide the GPU well
    // (at least 200 of the 256 units busy): a second co-resident workgroup buys little there and doubles the
    // slabs the next kernel has to read.  Otherwise two per compute unit.  (At M = 100 matrices with few column
    // units still take up to 16 slices: idle compute units cost more than the slab traffic.)
    constexpr int capacity = 512;
    int ks = (int)(capacity / 2 / tiles);
    if (ks < 1 || tiles * ks < 200) ks = (int)(capacity / tiles);
    int cap = GEMM_KSCAP / (p.M > 0 ? p.M : 1);
    if (cap > SMH_MAX_KSPLIT) cap = SMH_MAX_KSPLIT;
    if (ks > cap) ks = cap;
    if (ks > steps / GEMM_STAGES) ks = steps / GEMM_STAGES;
    if (ks < 1) ks = 1;
    p.steps_per_slice = (steps + ks - 1) / ks;
    p.ksplit = (steps + p.steps_per_slice - 1) / p.steps_per_slice;
    // Range cut: a launch that would put two workgroups on some compute units and one on others (256 < workgroups <= 512)
    // deals runs of steps instead, one workgroup per compute unit, crossing unit boundaries.
    p.chunk = 0;
    const long wgs = tiles * p.ksplit;
    if (p.mblocks == 1 && p.K % 32 == 0 && wgs > 256 && wgs <= 512) {
        const long total = (long)p.units * steps;
        const int chunk = (int)((total + 255) / 256);
        if (chunk <= steps && chunk >= 2 * GEMM_STAGES) {
            int pieces = 0;
            for (int u = 0; u < p.units; ++u) {
                const int n = (int)(((long)u * steps + steps - 1) / chunk - ((long)u * steps) / chunk) + 1;
                if (n > pieces) pieces = n;
            }
            if (pieces <= p.ksplit) {           // never more slabs than the even split leaves
                p.chunk = chunk;
                p.ksplit = pieces;
                p.steps_per_slice = chunk;
            }
        }
    }
}

typedef void (*gemm_kernel_t)(MatmulParams);

template <bool TILED>
static int gemm_launch_layout(const MatmulParams &p, hipStream_t stream) {
    // one instantiation per number of 16-row tiles (M <= 128) keeps the step free of branches; K % 32 != 0
    // takes the masked variant with all 8 tiles
    constexpr int W = TILED ? GEMM_TILED_WAVES : GEMM_WAVES;
    static const gemm_kernel_t exact[9] = {nullptr, q40_gemm_kernel<2, false, TILED, W>, q40_gemm_kernel<2, false, TILED, W>,
                                           q40_gemm_kernel<3, false, TILED, W>, q40_gemm_kernel<4, false, TILED, W>,
                                           q40_gemm_kernel<5, false, TILED, W>, q40_gemm_kernel<6, false, TILED, W>,
                                           q40_gemm_kernel<7, false, TILED, W>, q40_gemm_kernel<8, false, TILED, W>};
    // one workgroup per compute unit: the variant with the DMA wave
    constexpr bool HAS_DMA_WAVE = W == 8;
    constexpr int PS = HAS_DMA_WAVE ? GEMM_DMA_WAVE_SLOTS : GEMM_STAGES;
    static const gemm_kernel_t with_dma_wave[9] = {
        nullptr, q40_gemm_kernel<2, false, TILED, W, PS, HAS_DMA_WAVE>, q40_gemm_kernel<2, false, TILED, W, PS, HAS_DMA_WAVE>,
        q40_gemm_kernel<3, false, TILED, W, PS, HAS_DMA_WAVE>, q40_gemm_kernel<4, false, TILED, W, PS, HAS_DMA_WAVE>,
        q40_gemm_kernel<5, false, TILED, W, PS, HAS_DMA_WAVE>, q40_gemm_kernel<6, false, TILED, W, PS, HAS_DMA_WAVE>,
        q40_gemm_kernel<7, false, TILED, W, PS, HAS_DMA_WAVE>, q40_gemm_kernel<8, false, TILED, W, PS, HAS_DMA_WAVE>};
    static const gemm_kernel_t range_cut[9] = {
        nullptr, q40_gemm_kernel<2, false, TILED, W, PS, HAS_DMA_WAVE, true>, q40_gemm_kernel<2, false, TILED, W, PS, HAS_DMA_WAVE, true>,
        q40_gemm_kernel<3, false, TILED, W, PS, HAS_DMA_WAVE, true>, q40_gemm_kernel<4, false, TILED, W, PS, HAS_DMA_WAVE, true>,
        q40_gemm_kernel<5, false, TILED, W, PS, HAS_DMA_WAVE, true>, q40_gemm_kernel<6, false, TILED, W, PS, HAS_DMA_WAVE, true>,
        q40_gemm_kernel<7, false, TILED, W, PS, HAS_DMA_WAVE, true>, q40_gemm_kernel<8, false, TILED, W, PS, HAS_DMA_WAVE, true>};
    static const gemm_kernel_t ragged = q40_gemm_kernel<8, true, TILED, 4>;
    // more than 64 KB of dynamic LDS has to be allowed once per kernel (the attribute is not stream work,
    // so a launch under graph capture is not affected)
    static const hipError_t lds_ok = [] {
        hipError_t e = hipFuncSetAttribute((const void *)ragged, hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_LDS);
        for (int t = 2; t <= 8 && e == hipSuccess; ++t)
            e = hipFuncSetAttribute((const void *)exact[t], hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_LDS);
        for (int t = 2; t <= 8 && e == hipSuccess && HAS_DMA_WAVE; ++t)
            e = hipFuncSetAttribute((const void *)with_dma_wave[t], hipFuncAttributeMaxDynamicSharedMemorySize, PS * GS_BYTES);
        for (int t = 2; t <= 8 && e == hipSuccess; ++t)
            e = hipFuncSetAttribute((const void *)range_cut[t], hipFuncAttributeMaxDynamicSharedMemorySize, PS * GS_BYTES);
        return e;
    }();
    if (lds_ok != hipSuccess) {
        set_error("q40 gemm: the kernels' LDS could not be reserved: %s", hipGetErrorString(lds_ok));
        return (int)lds_ok;
    }
    SMH_REQUIRE((long)p.M * p.lda * 2 < (1L << 32), "q40 gemm: M x lda = %d x %ld exceeds the 32-bit lane offsets of A", p.M, p.lda);
    const int tiles = p.mblocks > 1 ? p.block_rows / 16 : (p.M + 15) / 16;
    const bool one_each = HAS_DMA_WAVE && p.K % 32 == 0 && (p.chunk > 0 || (long)p.units * p.mblocks * p.ksplit <= GEMM_DMA_WAVE_MAX_WGS);
    const gemm_kernel_t kern = (p.K % 32 != 0) ? ragged : (p.chunk > 0 ? range_cut : one_each ? with_dma_wave : exact)[tiles < 2 ? 2 : tiles];
    const long total_steps = (long)p.units * ((p.K + 31) / 32);
    dim3 grid((unsigned)(p.chunk > 0 ? (total_steps + p.chunk - 1) / p.chunk : (long)p.units_pad * p.mblocks * p.ksplit));
    hipLaunchKernelGGL(kern, grid, dim3(kern == ragged ? GEMM_THREADS : 64 * W + (one_each ? 64 : 0)), one_each ? PS * GS_BYTES : GEMM_LDS, stream, p);
    return launch_status();
}

typedef void (*gemm_kg_kernel_t)(MatmulParams);
static int gemm_kg_launch(const MatmulParams &p, hipStream_t stream) {
    static const gemm_kg_kernel_t kern[9] = {nullptr, nullptr, q40_gemm_kg_kernel<2>, q40_gemm_kg_kernel<3>, q40_gemm_kg_kernel<4>, q40_gemm_kg_kernel<5>,
                                             q40_gemm_kg_kernel<6>, q40_gemm_kg_kernel<7>, q40_gemm_kg_kernel<8>};
    static const int lds_bytes[9] = {0, 0, KgShape<2>::LDS, KgShape<3>::LDS, KgShape<4>::LDS, KgShape<5>::LDS, KgShape<6>::LDS, KgShape<7>::LDS, KgShape<8>::LDS};
    static const hipError_t lds_ok = [] {
        hipError_t e = hipSuccess;
        for (int t = 2; t <= 8 && e == hipSuccess; ++t)
            e = hipFuncSetAttribute((const void *)kern[t], hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes[t]);
        return e;
    }();
    if (lds_ok != hipSuccess) {
        set_error("q40 gemm: the kernels' LDS could not be reserved: %s", hipGetErrorString(lds_ok));
        return (int)lds_ok;
    }
    SMH_REQUIRE((long)p.M * p.lda * 2 < (1L << 32), "q40 gemm: M x lda = %d x %ld exceeds the 32-bit lane offsets of A", p.M, p.lda);
    int tiles = p.mblocks > 1 ? p.block_rows / 16 : (p.M + 15) / 16;
    if (tiles < 2) tiles = 2;
    dim3 grid((unsigned)(2L * p.units_pad * p.mblocks * p.ksplit));
    hipLaunchKernelGGL(kern[tiles], grid, dim3(576), lds_bytes[tiles], stream, p);
    return launch_status();
}

// Can w1|w3 of these dimensions run with SwiGLU inside the launch, and is it the faster way?  17 .. 128 rows, K a multiple of
// 64, two weights of n_half columns (a multiple of 128) whose 2 * n_half / 128 workgroups fit the compute units in one round;
// `worth_it`: and fill at least half of them (narrower weights are faster as two kernels with a K-split), above 32 rows
// (measured at the 7B shape, w1|w3 + SiLU: 38.1 against 44.9 us at 100 rows, 29.1 against 31.5 at 64, level at 32).
bool gemm_swiglu_fits(int M, int K, int n_half, bool worth_it) {
    if (M <= SMH_GEMV_MAX_M || M > 128 || K <= 0 || K % 64 != 0 || n_half <= 0 || n_half % 128 != 0) return false;
    const int wgs = 2 * (n_half / 128);
    return wgs <= 256 && (!worth_it || (wgs >= 128 && M > 32));
}

typedef void (*gemm_swiglu_kernel_t)(MatmulParams);
int gemm_swiglu_launch(const MatmulParams &p, hipStream_t stream) {
    static const gemm_swiglu_kernel_t kern[9] = {nullptr, nullptr, q40_gemm_swiglu_kernel<2>, q40_gemm_swiglu_kernel<3>, q40_gemm_swiglu_kernel<4>,
                                                 q40_gemm_swiglu_kernel<5>, q40_gemm_swiglu_kernel<6>, q40_gemm_swiglu_kernel<7>,
                                                 q40_gemm_swiglu_kernel<8>};
    static const int lds_bytes[9] = {0, 0, SwigluShape<2>::LDS, SwigluShape<3>::LDS, SwigluShape<4>::LDS, SwigluShape<5>::LDS, SwigluShape<6>::LDS,
                                     SwigluShape<7>::LDS, SwigluShape<8>::LDS};
    static const hipError_t lds_ok = [] {
        hipError_t e = hipSuccess;
        for (int t = 2; t <= 8 && e == hipSuccess; ++t)
            e = hipFuncSetAttribute((const void *)kern[t], hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes[t]);
        return e;
    }();
    if (lds_ok != hipSuccess) {
        set_error("q40 gemm: the kernels' LDS could not be reserved: %s", hipGetErrorString(lds_ok));
        return (int)lds_ok;
    }
    SMH_REQUIRE((long)p.M * p.lda * 2 < (1L << 32), "q40 gemm: M x lda = %d x %ld exceeds the 32-bit lane offsets of A", p.M, p.lda);
    int tiles = (p.M + 15) / 16;
    if (tiles < 2) tiles = 2;
    hipLaunchKernelGGL(kern[tiles], dim3((unsigned)(2 * (p.seg[0].N / 128))), dim3(576), lds_bytes[tiles], stream, p);
    return launch_status();
}

int gemm_launch(const MatmulParams &p, hipStream_t stream) {
    if (p.kgroups == 2 && p.tiled) return gemm_kg_launch(p, stream);
    return p.tiled ? gemm_launch_layout<true>(p, stream) : gemm_launch_layout<false>(p, stream);
}

}  // namespace smh

