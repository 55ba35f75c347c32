// Shared host/device declarations of the Q4_0 matmul kernels (GEMV for M <= 16, GEMM above).
//
// Both kernels cut K into slices for occupancy and write one [M, n_total] slab per slice into
// the caller's `partial` buffer; the slabs are added in slice order (in fp32) by the consuming kernel
// (partial_ops.hip).  With a single slice and a plain epilogue the product is written directly.
// Slabs of a product with at most SMH_GEMV_MAX_M rows hold fp32; above that they hold fp16: at those
// batch sizes writing and re-reading the slabs costs as much HBM traffic as the weights themselves,
// and a partial sum rounded to fp16 carries the same relative error as the fp16 result it ends up in.
#pragma once

#include "smh_common.hpp"

#define SMH_MAX_KSPLIT 16
#define SMH_MAX_SEGMENTS 3

#include "matmul_finish.hpp"

namespace smh {

struct MatmulSegment {
    const uint8_t *w;    // packed nibbles [K, N/2]
    const half_t *s;     // scales [K, N/64]
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
    int mblocks;             // GEMM: 128-row blocks
    int ksplit, steps_per_slice;
    int epilogue, direct;
    int slab_half;           // slabs hold fp16 instead of fp32 (see slab_is_half)
    MatmulFinish fin;        // fin.mode == 0: leave the slabs to another launch
};

__device__ __forceinline__ half_t matmul_epilogue(const MatmulParams &p, float acc, int m, int n) {
    half_t v = (half_t)acc;
    if (p.epilogue == SMH_EPI_RESIDUAL) v = (half_t)((float)p.resid[(long)m * p.ldr + n] + (float)v);
    return v;
}

// The dtype of the slabs follows from the row count alone, so producer and consumer agree without a flag.
__host__ __device__ inline bool slab_is_half(int M) { return M > SMH_GEMV_MAX_M; }

int env_int(const char *name, int dflt);
void gemv_fill_plan(MatmulParams &p);
int gemv_launch(const MatmulParams &p, hipStream_t stream);
void gemm_fill_plan(MatmulParams &p);
int gemm_launch(const MatmulParams &p, hipStream_t stream);

}  // namespace smh
