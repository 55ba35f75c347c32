// Shared host/device declarations of the Q4_0 matmul kernels (GEMV for M <= 16, GEMM above).
//
// Both kernels cut K into slices for occupancy and write one [M, n_total] slab per slice into
// the caller's `partial` buffer; the slabs are added in slice order (in fp32) by the consuming kernel
// (partial_ops.hip).  With a single slice and a plain epilogue the product is written directly.
// The slabs hold fp32 at every batch size.
#pragma once

#include "smh_common.hpp"

#define SMH_MAX_KSPLIT 16
#define SMH_MAX_SEGMENTS 3
#define SMH_SILU_IN_MAX_M 2
#define SMH_SILU_IN_MAX_K 2048      /* rows of a K-slice whose activations fit the workgroup's LDS */
#define SMH_NORM_SUMS 16            /* partial sums of squares per row that smh_partial_residual_sumsq leaves */
#define SMH_NORM_IN_MAX_XS_BYTES 28160   /* M x K-slice fp16 activations next to the weight rings, two workgroups per CU */

namespace smh {

// ---- tiled weight layout ---------------------------------------------------------------------------
// The checkpoint layout (bytes [K, N/2], scales [K, N/64]) costs the matmul kernels one cache-line request
// per k-row for the scales of a 256-column unit (8 bytes out of a 128-byte line) - as many requests as the
// nibbles need - and byte permutes to bring 8 consecutive k of one column into a lane.  smh_q40_tile
// rewrites a weight once into the order the kernels consume it:
//   tiled[unit][step] = one contiguous tile of TILE_BYTES for 256 columns x 32 rows:
//     TILE_W_BYTES of nibbles as [piece q = 0..3][lane = 16 g + c][4 dwords]: piece q = 2 blk + B / 2 holds,
//       for byte column 64 blk + 4 c + B of the checkpoint row (B = 2 (q & 1) and 2 (q & 1) + 1) and rows
//       r_i = 32 step + 8 g + i, the dwords x = bytes (r0, r4, r1, r5) and x2 = (r2, r6, r3, r7), every byte
//       XORed with 0x88 (two's-complement nibble -> code + 8).  (x, x2, x >> 8, x2 >> 8) then carry the
//       row pairs (0,1), (2,3), (4,5), (6,7) in bytes 0 and 2: the register layout of an MFMA B operand
//       (lane = column, 8 consecutive k) is two shifts and eight AND-ORs away.
//     TILE_S_BYTES of scales as [g][group = 0..3][i = 0..7] fp16: the 8 rows of k-octet g for each of the
//       unit's four 64-column groups, i.e. the factors of one A operand in its register order.
//   Columns past N and rows past K are filled with code 0 and scale 0 (they contribute exact zeros).
constexpr int TILE_W_BYTES = 4096;
constexpr int TILE_S_BYTES = 256;
constexpr int TILE_BYTES = TILE_W_BYTES + TILE_S_BYTES;
__host__ __device__ inline long tiled_units(int N) { return (N + 255) / 256; }
__host__ __device__ inline long tiled_steps(int K) { return (K + 31) / 32; }

struct MatmulSegment {
    const uint8_t *w;    // packed nibbles [K, N/2]; tiled: the tiles of this weight
    const half_t *s;     // scales [K, N/64]; tiled: unused
    int N;               // columns of this weight
    int col0;            // first output column
    int unit0;           // first work unit (column pair / column block) of this weight
};

struct MatmulParams {
    const half_t *a;
    half_t *c;               // direct output (ksplit == 1)
    const half_t *resid;
    float *partial;          // [ksplit][M][n_total]
    MatmulSegment seg[SMH_MAX_SEGMENTS];
    long lda, ldc, ldr;
    int M, K;
    int nseg, n_total;
    int units, units_pad;    // column units over all segments (GEMV: padded to a multiple of 8)
    int mblocks, block_rows; // GEMM: row blocks and the rows of one (128, or 64 where two blocks of a narrow matrix halve its K-slices)
    int ksplit, steps_per_slice;
    int kgroups;             // GEMM, 2: q40_gemm_kg_kernel (128-column blocks, two K-groups a workgroup)
    int chunk;               // GEMM, > 0: range cut - workgroup j takes steps [j * chunk, (j + 1) * chunk) of the column units laid end to end
    int epilogue, direct;
    int tiled;               // the segments' weights are in the tiled layout
    // GEMV, at most SMH_SILU_IN_MAX_M rows: the activations are not read from `a` but made by every workgroup for
    // its own K-slice from the slabs of the gate|up product, a[m][k] = silu(gate[m][k]) * up[m][k] (gate = columns
    // 0..K-1, up = columns K..2K-1 of the slabs), with the roundings of partial_silu_mul_kernel
    const float *gu_partial;
    int gu_ksplit;
    // GEMV, norm_w != nullptr: `a` holds the un-normalised residual stream h; every workgroup makes its K-slice of
    // RMSNorm(h) * norm_w itself, a[m][k] = fp16(fp16(h[m][k] * r[m]) * norm_w[k]) with r[m] = 1 / sqrt(sum / K + eps)
    // and sum = norm_ss[m][0] + ... + norm_ss[m][SMH_NORM_SUMS - 1] added in that order (partial_rmsnorm_kernel's roundings)
    const half_t *norm_w;
    const float *norm_ss;
    float norm_eps;
};

__device__ __forceinline__ half_t matmul_epilogue(const MatmulParams &p, float acc, int m, int n) {
    half_t v = (half_t)acc;
    if (p.epilogue == SMH_EPI_RESIDUAL) v = (half_t)((float)p.resid[(long)m * p.ldr + n] + (float)v);
    return v;
}

void gemv_fill_plan(MatmulParams &p);
int gemv_launch(const MatmulParams &p, hipStream_t stream);
bool gemv_norm_in_fits(const MatmulParams &p);     // after gemv_fill_plan: can RMSNorm be made inside the launch
void gemm_fill_plan(MatmulParams &p);
int gemm_launch(const MatmulParams &p, hipStream_t stream);
bool gemm_swiglu_fits(int M, int K, int n_half, bool worth_it);
int gemm_swiglu_launch(const MatmulParams &p, hipStream_t stream);     // seg[0] = gate, seg[1] = up (tiled), c / ldc = the activations

}  // namespace smh
