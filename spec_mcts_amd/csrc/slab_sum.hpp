// Sums over the K-slice slabs a Q4_0 matmul kernel leaves (q40_matmul.hpp), in slice order, in fp32.
#pragma once

#include "q40_matmul.hpp"

namespace smh {

// Element `idx` of every slab, added in slice order in fp32.  `half`: the slabs hold fp16 (slab_is_half).
__device__ __forceinline__ float slab_sum(const void *partial, long idx, long slab_stride, int ksplit, bool half) {
    float v[SMH_MAX_KSPLIT];
    if (half) {
        const half_t *p = reinterpret_cast<const half_t *>(partial) + idx;
#pragma unroll
        for (int s = 0; s < SMH_MAX_KSPLIT; ++s) v[s] = (s < ksplit) ? (float)p[s * slab_stride] : 0.f;
    } else {
        const float *p = reinterpret_cast<const float *>(partial) + idx;
#pragma unroll
        for (int s = 0; s < SMH_MAX_KSPLIT; ++s) v[s] = (s < ksplit) ? p[s * slab_stride] : 0.f;
    }
    float tot = 0.f;
#pragma unroll
    for (int s = 0; s < SMH_MAX_KSPLIT; ++s) tot += v[s];
    return tot;
}
// Two consecutive elements (idx % 2 == 0).
__device__ __forceinline__ f2 slab_sum2(const void *partial, long idx, long slab_stride, int ksplit, bool half) {
    f2 tot = {0.f, 0.f};
    if (half) {
        const half_t *p = reinterpret_cast<const half_t *>(partial) + idx;
        h2 v[SMH_MAX_KSPLIT];
#pragma unroll
        for (int s = 0; s < SMH_MAX_KSPLIT; ++s)
            v[s] = (s < ksplit) ? *reinterpret_cast<const h2 *>(p + s * slab_stride) : h2{(half_t)0.f, (half_t)0.f};
#pragma unroll
        for (int s = 0; s < SMH_MAX_KSPLIT; ++s) { tot[0] += (float)v[s][0]; tot[1] += (float)v[s][1]; }
    } else {
        const float *p = reinterpret_cast<const float *>(partial) + idx;
        f2 v[SMH_MAX_KSPLIT];
#pragma unroll
        for (int s = 0; s < SMH_MAX_KSPLIT; ++s)
            v[s] = (s < ksplit) ? *reinterpret_cast<const f2 *>(p + s * slab_stride) : f2{0.f, 0.f};
#pragma unroll
        for (int s = 0; s < SMH_MAX_KSPLIT; ++s) tot += v[s];
    }
    return tot;
}
// Four consecutive elements (idx % 4 == 0).
__device__ __forceinline__ f4 slab_sum4(const void *partial, long idx, long slab_stride, int ksplit, bool half) {
    f4 tot = {0.f, 0.f, 0.f, 0.f};
    if (half) {
        const half_t *p = reinterpret_cast<const half_t *>(partial) + idx;
        h4 v[SMH_MAX_KSPLIT];
#pragma unroll
        for (int s = 0; s < SMH_MAX_KSPLIT; ++s)
            v[s] = (s < ksplit) ? *reinterpret_cast<const h4 *>(p + s * slab_stride) : h4{(half_t)0.f, (half_t)0.f, (half_t)0.f, (half_t)0.f};
#pragma unroll
        for (int s = 0; s < SMH_MAX_KSPLIT; ++s)
#pragma unroll
            for (int j = 0; j < 4; ++j) tot[j] += (float)v[s][j];
    } else {
        const float *p = reinterpret_cast<const float *>(partial) + idx;
        f4 v[SMH_MAX_KSPLIT];
#pragma unroll
        for (int s = 0; s < SMH_MAX_KSPLIT; ++s)
            v[s] = (s < ksplit) ? *reinterpret_cast<const f4 *>(p + s * slab_stride) : f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < SMH_MAX_KSPLIT; ++s) tot += v[s];
    }
    return tot;
}

}  // namespace smh
