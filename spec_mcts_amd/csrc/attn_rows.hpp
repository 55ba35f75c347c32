// Row-at-a-time attention arithmetic shared by the decode attention kernels: a 16-lane group owns one
// K/V row of a 128-wide head, scores it against a query held in the same layout and folds it into an
// online-softmax state (base-2 exponentials; the caller pre-scales scores by log2(e)/sqrt(D)).
#pragma once

#include "smh_common.hpp"

namespace smh {

// ---- suffix rows ----------------------------------------------------------------------------------------
// A 16-lane group handles one row at a time; lane c of the group owns head dims 4c..4c+3 ("low half")
// and 64+4c..64+4c+3 ("high half"), held as fp16 pairs in the order (0,2),(1,3) that nibble decoding
// produces.
struct RowRegs { h2 a02, a13, b02, b13; };   // a: dims 4c.., b: dims 64+4c..

__device__ __forceinline__ RowRegs row_from_fp16(const half_t *row, int c) {
    const u32x2 lo = *reinterpret_cast<const u32x2 *>(row + 4 * c);
    const u32x2 hi = *reinterpret_cast<const u32x2 *>(row + 64 + 4 * c);
    RowRegs r;
    r.a02 = as_h2(pack_lo16(lo[0], lo[1]));
    r.a13 = as_h2(pack_hi16(lo[0], lo[1]));
    r.b02 = as_h2(pack_lo16(hi[0], hi[1]));
    r.b13 = as_h2(pack_hi16(hi[0], hi[1]));
    return r;
}
// bytes: this lane's dword of the packed row; sc: (scale of dims 0..63, scale of dims 64..127)
__device__ __forceinline__ RowRegs row_from_q40(uint32_t bytes, uint32_t sc) {
    const uint32_t u = bytes ^ NIBBLE_FLIP, u1 = u >> 8;
    const h2 s_a = as_h2(pack_lo16(sc, sc)), s_b = as_h2(pack_hi16(sc, sc));
    RowRegs r;
    r.a02 = codes_high(u) * s_a;
    r.a13 = codes_high(u1) * s_a;
    r.b02 = codes_low(u) * s_b;
    r.b13 = codes_low(u1) * s_b;
    return r;
}
__device__ __forceinline__ float row_dot(const RowRegs &k, const RowRegs &q) {
    float s = __builtin_amdgcn_fdot2(k.a02, q.a02, 0.f, false);
    s = __builtin_amdgcn_fdot2(k.a13, q.a13, s, false);
    s = __builtin_amdgcn_fdot2(k.b02, q.b02, s, false);
    s = __builtin_amdgcn_fdot2(k.b13, q.b13, s, false);
    return row16_sum(s);
}

struct SoftState {
    float m, l;
    float o[8];     // dims 4c+0, 4c+2, 4c+1, 4c+3, 64+4c+0, 64+4c+2, 64+4c+1, 64+4c+3
};
__device__ __forceinline__ void soft_add_row(SoftState &st, float score, const RowRegs &v) {
    const float m_new = fmaxf(st.m, score);
    const float corr = exp2f(st.m - m_new);          // st.m = -inf on first use: exp2(-inf) = 0
    const float pr = exp2f(score - m_new);
    st.m = m_new;
    st.l = st.l * corr + pr;
    st.o[0] = st.o[0] * corr + pr * (float)v.a02.x;
    st.o[1] = st.o[1] * corr + pr * (float)v.a02.y;
    st.o[2] = st.o[2] * corr + pr * (float)v.a13.x;
    st.o[3] = st.o[3] * corr + pr * (float)v.a13.y;
    st.o[4] = st.o[4] * corr + pr * (float)v.b02.x;
    st.o[5] = st.o[5] * corr + pr * (float)v.b02.y;
    st.o[6] = st.o[6] * corr + pr * (float)v.b13.x;
    st.o[7] = st.o[7] * corr + pr * (float)v.b13.y;
}
// fold an un-normalised partial (m2, l2, o2) into st
__device__ __forceinline__ void soft_merge(SoftState &st, float m2, float l2, const float *o2) {
    const float m_new = fmaxf(st.m, m2);
    if (m_new == -INFINITY) return;                  // both empty
    const float c1 = exp2f(st.m - m_new), c2 = exp2f(m2 - m_new);
    st.m = m_new;
    st.l = st.l * c1 + l2 * c2;
#pragma unroll
    for (int j = 0; j < 8; ++j) st.o[j] = st.o[j] * c1 + o2[j] * c2;
}

}  // namespace smh
