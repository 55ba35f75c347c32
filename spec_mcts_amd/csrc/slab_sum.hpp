// Sums over the K-slice slabs a Q4_0 matmul kernel leaves (q40_matmul.hpp), in slice order, in fp32.
#pragma once

#include "q40_matmul.hpp"

namespace smh {

// Element `idx` of every slab (fp32), added in slice order.
__device__ __forceinline__ float slab_sum(const void *partial, long idx, long slab_stride, int ksplit) {
    const float *p = reinterpret_cast<const float *>(partial) + idx;
    float v[SMH_MAX_KSPLIT];
#pragma unroll
    for (int s = 0; s < SMH_MAX_KSPLIT; ++s) v[s] = (s < ksplit) ? p[s * slab_stride] : 0.f;
    float tot = 0.f;
#pragma unroll
    for (int s = 0; s < SMH_MAX_KSPLIT; ++s) tot += v[s];
    return tot;
}
// Two consecutive elements (idx % 2 == 0).
__device__ __forceinline__ f2 slab_sum2(const void *partial, long idx, long slab_stride, int ksplit) {
    const float *p = reinterpret_cast<const float *>(partial) + idx;
    f2 v[SMH_MAX_KSPLIT];
#pragma unroll
    for (int s = 0; s < SMH_MAX_KSPLIT; ++s) v[s] = (s < ksplit) ? *reinterpret_cast<const f2 *>(p + s * slab_stride) : f2{0.f, 0.f};
    f2 tot = {0.f, 0.f};
#pragma unroll
    for (int s = 0; s < SMH_MAX_KSPLIT; ++s) tot += v[s];
    return tot;
}
// Four consecutive elements (idx % 4 == 0).
__device__ __forceinline__ f4 slab_sum4(const void *partial, long idx, long slab_stride, int ksplit) {
    const float *p = reinterpret_cast<const float *>(partial) + idx;
    f4 v[SMH_MAX_KSPLIT];
#pragma unroll
    for (int s = 0; s < SMH_MAX_KSPLIT; ++s) v[s] = (s < ksplit) ? *reinterpret_cast<const f4 *>(p + s * slab_stride) : f4{0.f, 0.f, 0.f, 0.f};
    f4 tot = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < SMH_MAX_KSPLIT; ++s) tot += v[s];
    return tot;
}

}  // namespace smh
