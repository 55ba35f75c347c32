// One decode step of the Q4_0 transformer for up to 16 branches as ONE persistent kernel.
//
// At 1..16 rows per step every matrix of the model is read exactly once per step and nothing else
// is large, so the step is bound by how steadily the packed weights stream out of HBM.  A chain of
// one kernel per operator drains and refills the memory pipeline some 400 times per step; here one
// workgroup per compute unit stays resident for the whole step and
//   * its 4 STREAM waves own private rings of 32-row weight steps in LDS, filled by direct-to-LDS
//     loads.  Weights do not depend on activations, so every wave knows the complete sequence of
//     steps it will need (over all phases of all layers) and keeps its ring full ACROSS phase
//     boundaries: HBM keeps streaming while the workgroups synchronise;
//   * its 4 CONTROL waves do everything that waits for other workgroups: the grid barrier, loading
//     the phase's activations into LDS, publishing partial sums and finishing a 256-column unit
//     when the last partial of the unit has arrived.  Stream waves never wait for a global memory
//     round trip except their own ring.
//
// Phases of a layer (a grid barrier after each):
//   QKV   x = RMSNorm(h)            . [wq|wk|wv]   finisher: RoPE, q / exact k,v out, Q4_0 KV append
//   ATT   softmax(q K^T) V over the shared fp16 prefix (in chunks) and the branch's Q4_0 suffix
//   O     x = attention output     . wo          finisher: h += fp16(sum), sum of squares of h
//   W13   x = RMSNorm(h)            . [w1|w3]     finisher: fp16(silu(gate)) * up
//   W2    x = SiLU product          . w2          finisher: h += fp16(sum), sum of squares of h
//
// Work split of a matrix phase: the units x (K/32) steps of the phase form one line, cut into equal
// ranges, one per workgroup (so a workgroup touches at most two units); the 4 stream waves take the
// steps of the range round-robin.  Per unit the waves' accumulators are folded through LDS, the
// control waves write the workgroup's partial (fp32 [M,256]) and count the arrival; the workgroup
// whose arrival completes the unit adds the partials in workgroup order (results do not depend on
// timing) and applies the operator that follows the matrix in the model, rounding where the
// module-by-module path rounds.
//
// Data that one workgroup writes and another reads inside the launch travels as device-scope
// relaxed atomics (write-through stores, cache-bypassing loads); every wait is bounded: a spin that
// runs out sets an error word, after which all waits fall through and the kernel drains.
#include <stdlib.h>

#include <map>
#include <mutex>

#include "attn_rows.hpp"
#include "rope_kv.hpp"

#ifdef SMH_MEGA_DEBUG
__device__ unsigned long long smh_mega_trace[8][4096];
#define MTR(slotbase, k) do { if (trace_on && lane0 == 0) smh_mega_trace[slotbase][trace_i++ & 4095] = ((unsigned long long)(k) << 56) | (__builtin_readcyclecounter() & 0xFFFFFFFFFFFFFFull); } while (0)
#else
#define MTR(slotbase, k) do {} while (0)
#endif
namespace smh {

int env_int(const char *name, int dflt);

constexpr int MK_STREAM_WAVES = 4;
constexpr int MK_CONTROL_WAVES = 4;
constexpr int MK_THREADS = (MK_STREAM_WAVES + MK_CONTROL_WAVES) * 64;
constexpr int MK_STAGE_W = 32 * 128;                 // 32 rows x 128 bytes of packed nibbles
constexpr int MK_STAGE_S = 32 * 8;                   // 32 rows x 4 scales
constexpr int MK_STAGE = MK_STAGE_W + MK_STAGE_S;
constexpr int MK_MAX_STAGES = 8;
constexpr int MK_MAX_M = 16;
constexpr int MK_PART = 132;                         // floats per attention partial: o[128], m, l, pad
constexpr int MK_LDS_LIMIT = 160 * 1024;
constexpr int MK_SYNC_BYTES = 2048;                  // status words + barrier counters at the head of the workspace

enum { MK_QKV = 0, MK_O = 1, MK_W13 = 2, MK_W2 = 3, MK_MATRIX_PHASES = 4 };
enum { MK_X_NORM_ATTN = 0, MK_X_ATTN_OUT = 1, MK_X_NORM_FFN = 2, MK_X_ACT = 3 };

struct MegaLayer {                 // one per layer, in device memory; matrices in the order wq wk wv wo w1 w3 w2
    const uint8_t *w[7];
    const half_t *s[7];
    const half_t *attn_norm, *ffn_norm;
    const half_t *prefix_k, *prefix_v;          // [P][Hkv*128] fp16
    uint8_t *cache_k, *cache_v;                 // [B][Smax][Hkv][64]
    half_t *cache_ks, *cache_vs;                // [B][Smax][Hkv][2]
};

struct MegaMatrix {                // geometry of one matrix phase, the same for every layer
    int nseg, seg_id[3], seg_n[3], unit0[3];
    int K, steps, units, T, geff;
};

struct MegaParams {
    const MegaLayer *layers;
    const int64_t *tokens;
    const half_t *emb;
    const half_t *cos_tab, *sin_tab;
    const int32_t *pos_dev, *t_dev;
    half_t *h;                      // [M][dim] residual stream; holds the final hidden state at exit
    half_t *q, *cur_k, *cur_v;      // [M][H*128], [M][Hkv*128] x2
    half_t *attn_out;               // [M][H*128]
    half_t *act;                    // [M][ffn]
    float *slabs;                   // [G][2][M][256]
    float *ssq;                     // [2][dim/256][M]
    float *att_part;                // [H*(C+1)][M][MK_PART]
    uint32_t *unit_cnt;             // [4 phases][max units][4 control waves]
    uint32_t *att_cnt;              // [H]
    uint32_t *sync;                 // [0] barrier arrivals, [1] arrivals before this launch, [2] error
    MegaMatrix mat[MK_MATRIX_PHASES];
    int n_layers, M, dim, H, Hkv, ffn, P, Smax, G;
    int stages, max_units, chunks;  // ring depth; counter stride; prefix chunks per head
    int att_rows;                   // prefix rows per attention item (multiple of 16)
    int xbuf_off, red_off, flag_off;// LDS layout (bytes)
    int mr;                         // row groups of 4: ceil(M/4)
    int spin_limit;
    float eps, scale_log2;
};

// The parameter block is read through the constant address space: its fields arrive by scalar loads
// when they are needed instead of occupying registers for the whole kernel, and tables in it can be
// indexed.  The host uploads it once per configuration (smh_decode_prepare).
typedef const __attribute__((address_space(4))) MegaParams CParams;
typedef const __attribute__((address_space(4))) MegaLayer CLayer;
__device__ __forceinline__ CLayer &layer_of(CParams &p, int layer) {
    return *reinterpret_cast<CLayer *>(reinterpret_cast<uintptr_t>(p.layers + layer));
}
__device__ __forceinline__ MegaMatrix matrix_of(CParams &p, int ph) {
    MegaMatrix g;
    g.nseg = p.mat[ph].nseg;
#pragma unroll
    for (int i = 0; i < 3; ++i) {
        g.seg_id[i] = p.mat[ph].seg_id[i];
        g.seg_n[i] = p.mat[ph].seg_n[i];
        g.unit0[i] = p.mat[ph].unit0[i];
    }
    g.K = p.mat[ph].K;
    g.steps = p.mat[ph].steps;
    g.units = p.mat[ph].units;
    g.T = p.mat[ph].T;
    g.geff = p.mat[ph].geff;
    return g;
}
__device__ __forceinline__ int sel3(int i, int v0, int v1, int v2) { return i == 0 ? v0 : i == 1 ? v1 : v2; }
__device__ __forceinline__ int pick3(const int (&v)[3], int i) { return sel3(i, v[0], v[1], v[2]); }

typedef const __attribute__((address_space(1))) void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;

// workgroup barrier that does not wait for the ring loads in flight (LDS traffic only)
__device__ __forceinline__ void wg_sync() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// ---- grid barrier (control waves) ------------------------------------------------------------------------
// A thousand atomics on one address take tens of microseconds, so arrivals go up a tree: the control
// waves of a workgroup count in LDS, the last of them increments the counter of the workgroup's group
// (16 groups, one cache line each), and the arrival that completes a group increments the top counter.
// Counters only grow; "complete" is a multiple of the group size.  One wave per workgroup polls the top
// counter and releases the other control waves through LDS.
// LDS words at flag_off: [0] attention finisher flag, [1] control-wave arrivals, [2] last barrier passed.
constexpr int MK_GROUPS = 16;
constexpr int MK_GROUP_WORD0 = 32, MK_GROUP_STRIDE = 16;      // uint32 index of group g's counter: 32 + 16 g
__device__ __forceinline__ void grid_arrive(CParams &p, uint32_t *words, int w, int lane) {
    wait_vmem();
    if (lane == 0) {
        const uint32_t old = __hip_atomic_fetch_add(words + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        if (((old + 1u) & (MK_CONTROL_WAVES - 1)) == 0u) {
            const int g = w & (MK_GROUPS - 1);
            const uint32_t size = (uint32_t)((p.G - g + MK_GROUPS - 1) / MK_GROUPS);
            const uint32_t prev = __hip_atomic_fetch_add(p.sync + MK_GROUP_WORD0 + MK_GROUP_STRIDE * g, 1u, __ATOMIC_RELAXED,
                                                         __HIP_MEMORY_SCOPE_AGENT);
            if ((prev + 1u) % size == 0u) __hip_atomic_fetch_add(p.sync, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}
__device__ __forceinline__ void grid_wait(CParams &p, uint32_t *words, int cw, uint32_t target, uint32_t barrier_no) {
    int it = 0;
    if (cw == 0) {
        while (true) {
            const uint32_t v = ld_u32(p.sync);
            if ((int32_t)(v - target) >= 0) break;
            if ((it & 63) == 63 && ld_u32(p.sync + 2) != 0u) break;
            if (++it > p.spin_limit) {
                st_u32(p.sync + 2, 1u);
                break;
            }
            __builtin_amdgcn_s_sleep(1);
        }
        __hip_atomic_store(words + 2, barrier_no, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    } else {
        while (true) {
            const uint32_t v = __hip_atomic_load(words + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            if ((int32_t)(v - barrier_no) >= 0) break;
            if (++it > p.spin_limit) break;
            __builtin_amdgcn_s_sleep(1);
        }
    }
}

// ---- geometry ----------------------------------------------------------------------------------------
__device__ __forceinline__ void wg_range(const MegaMatrix &g, int w, int &a, int &b) {
    if (w >= g.geff) {
        a = b = 0;
        return;
    }
    a = (int)((uint32_t)w * (uint32_t)g.T / (uint32_t)g.geff);
    b = (int)((uint32_t)(w + 1) * (uint32_t)g.T / (uint32_t)g.geff);
}
// workgroups that contribute to unit u: first..last
__device__ __forceinline__ void unit_contributors(const MegaMatrix &g, int u, int &first, int &last) {
    const uint32_t X = (uint32_t)u * g.steps, Y = X + g.steps;
    first = (int)(((X + 1) * (uint32_t)g.geff + g.T - 1) / (uint32_t)g.T) - 1;
    last = (int)((Y * (uint32_t)g.geff + g.T - 1) / (uint32_t)g.T) - 1;
}

// ---- the stream of weight steps of one wave -------------------------------------------------------------
// The position is kept as running addresses: issuing a step costs five loads and a few scalar adds;
// geometry and layer pointers are looked up only when the cursor enters a phase or a new unit.
struct Cursor {
    int layer, ph;          // layer, matrix phase
    int j, n;               // next step of the workgroup's range this wave takes; length of the range
    int unit, kstep, steps; // position of that step; steps per unit in this phase
    const uint8_t *wb, *sb; // nibbles / scales of row 32*kstep of the unit (uniform)
    uint32_t rowb, srow;    // row pitches in bytes
    uint32_t w_off, s_off;  // this lane's byte offsets inside a step
};
__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ const uint8_t *uni(const uint8_t *ptr) {
    const uint64_t v = reinterpret_cast<uint64_t>(ptr);
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
    return reinterpret_cast<const uint8_t *>(((uint64_t)hi << 32) | lo);
}
// addresses of the cursor's (layer, phase, unit, kstep)
__device__ __forceinline__ void cursor_locate(Cursor &c, CParams &p, int lane) {
    const MegaMatrix g = matrix_of(p, c.ph);
    int sg = 0;
    if (g.nseg > 1 && c.unit >= g.unit0[1]) sg = 1;
    if (g.nseg > 2 && c.unit >= g.unit0[2]) sg = 2;
    CLayer &L = layer_of(p, c.layer);
    const int id = pick3(g.seg_id, sg);
    const int N = pick3(g.seg_n, sg);
    const int ul = c.unit - pick3(g.unit0, sg);
    c.rowb = (uint32_t)uni(N / 2);
    c.srow = (uint32_t)uni(N / 32);
    c.wb = uni(L.w[id] + (long)c.kstep * 32 * c.rowb + (long)ul * 128);
    c.sb = uni(reinterpret_cast<const uint8_t *>(L.s[id]) + (long)c.kstep * 32 * c.srow + (long)ul * 8);
    c.w_off = (uint32_t)(lane >> 3) * c.rowb + 16u * (uint32_t)(lane & 7);
    c.s_off = (uint32_t)(lane >> 1) * c.srow + 4u * (uint32_t)(lane & 1);
}
__device__ __forceinline__ void cursor_enter(Cursor &c, CParams &p, int w, int wave, int lane) {
    const MegaMatrix g = matrix_of(p, c.ph);
    int a, b;
    wg_range(g, w, a, b);
    c.n = uni(b - a);
    c.j = wave;
    c.steps = uni(g.steps);
    const uint32_t t = (uint32_t)(a + wave);
    c.unit = uni((int)(t / (uint32_t)g.steps));
    c.kstep = uni((int)(t - (uint32_t)c.unit * g.steps));
    if (c.j < c.n) cursor_locate(c, p, lane);
}
// moves to the next phase until the cursor points at a step; false when the model is exhausted
__device__ __forceinline__ bool cursor_settle(Cursor &c, CParams &p, int w, int wave, int lane) {
    while (c.layer < p.n_layers && c.j >= c.n) {
        c.ph = uni(c.ph + 1);
        if (c.ph == MK_MATRIX_PHASES) {
            c.ph = 0;
            c.layer = uni(c.layer + 1);
        }
        if (c.layer < p.n_layers) cursor_enter(c, p, w, wave, lane);
    }
    return c.layer < p.n_layers;
}
// 5 direct-to-LDS loads: 4 x (8 rows x 128 B) of nibbles + 32 rows x 8 B of scales; then on to the wave's next step
__device__ __forceinline__ void cursor_issue(Cursor &c, CParams &p, uint8_t *stage, int lane) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
        __builtin_amdgcn_global_load_lds((gptr_t)(c.wb + (long)(8 * q) * c.rowb + c.w_off), (lptr_t)(stage + q * 1024), 16, 0, 0);
    __builtin_amdgcn_global_load_lds((gptr_t)(c.sb + c.s_off), (lptr_t)(stage + MK_STAGE_W), 4, 0, 0);
    c.j = uni(c.j + MK_STREAM_WAVES);
    c.kstep = uni(c.kstep + MK_STREAM_WAVES);
    if (c.kstep >= c.steps) {
        c.kstep = uni(c.kstep - c.steps);
        c.unit = uni(c.unit + 1);
        if (c.j < c.n) cursor_locate(c, p, lane);
    } else {
        c.wb = uni(c.wb + (long)(32 * MK_STREAM_WAVES) * c.rowb);
        c.sb = uni(c.sb + (long)(32 * MK_STREAM_WAVES) * c.srow);
    }
}

struct Ring {
    uint32_t base;                        // LDS byte offset of the wave's ring
    int stages, head, tail, inflight;     // head: next slot to consume; tail: next slot to fill
};
__device__ __forceinline__ void ring_fill(Ring &r, Cursor &c, CParams &p, uint8_t *lds, int w, int wave, int lane) {
    while (r.inflight < r.stages) {
        if (c.j >= c.n && !cursor_settle(c, p, w, wave, lane)) break;
        cursor_issue(c, p, lds + r.base + r.tail * MK_STAGE, lane);
        r.tail = uni((r.tail + 1 == r.stages) ? 0 : r.tail + 1);
        r.inflight = uni(r.inflight + 1);
    }
}
// wait until the oldest stage in flight has landed (loads complete in order)
__device__ __forceinline__ void ring_wait_head(const Ring &r) {
    switch (r.inflight) {
        case 8: asm volatile("s_waitcnt vmcnt(35)" ::: "memory"); break;
        case 7: asm volatile("s_waitcnt vmcnt(30)" ::: "memory"); break;
        case 6: asm volatile("s_waitcnt vmcnt(25)" ::: "memory"); break;
        case 5: asm volatile("s_waitcnt vmcnt(20)" ::: "memory"); break;
        case 4: asm volatile("s_waitcnt vmcnt(15)" ::: "memory"); break;
        case 3: asm volatile("s_waitcnt vmcnt(10)" ::: "memory"); break;
        case 2: asm volatile("s_waitcnt vmcnt(5)" ::: "memory"); break;
        default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    }
}

// ---- one 32-row step: decode + MFMA (offset codes, scales on the activation side) ------------------------
// acc tile t = (blk*2 + half)*4 + b holds column 128*blk + 64*half + 4c + b, rows 4g + r.
struct DecodeConsts {
    uint32_t mask_hi, mask_lo, magic_hi, magic_lo;
};
__device__ __forceinline__ void step_consume(const uint8_t *stage, const uint8_t *xt, int c, int g, int row, const DecodeConsts &C,
                                             f4 (&acc)[16], f4 (&corr)[4]) {
    uint32_t u0[8], u1[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        u0[i] = *reinterpret_cast<const uint32_t *>(stage + (8 * g + i) * 128 + 4 * c) ^ NIBBLE_FLIP;
        u1[i] = *reinterpret_cast<const uint32_t *>(stage + (8 * g + i) * 128 + 64 + 4 * c) ^ NIBBLE_FLIP;
    }
    const h8 xv = *reinterpret_cast<const h8 *>(xt + row * 64 + 16 * g);
    u32x2 sv[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) sv[i] = *reinterpret_cast<const u32x2 *>(stage + MK_STAGE_W + (8 * g + i) * 8);
    h8 a[4];
#pragma unroll
    for (int blk = 0; blk < 2; ++blk) {
        u32x4 s_hi, s_lo;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            s_hi[j] = pack_lo16(sv[2 * j][blk], sv[2 * j + 1][blk]);
            s_lo[j] = pack_hi16(sv[2 * j][blk], sv[2 * j + 1][blk]);
        }
        a[2 * blk] = xv * __builtin_bit_cast(h8, s_hi);
        a[2 * blk + 1] = xv * __builtin_bit_cast(h8, s_lo);
    }
    const h8 ones = {(half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f};
#pragma unroll
    for (int bh = 0; bh < 4; ++bh) corr[bh] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[bh], ones, corr[bh], 0, 0, 0);
#define SMH_MK_BYTE(U, BLK, B)                                                                                      \
    {                                                                                                               \
        u32x4 vh, vl;                                                                                               \
        _Pragma("unroll") for (int j = 0; j < 4; ++j) {                                                             \
            const uint32_t pr = pair_bytes<B>(U[2 * j], U[2 * j + 1]);                                              \
            vh[j] = (pr & C.mask_hi) | C.magic_hi;                                                                  \
            vl[j] = (pr & C.mask_lo) | C.magic_lo;                                                                  \
        }                                                                                                           \
        acc[(BLK * 2) * 4 + B] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[2 * BLK], __builtin_bit_cast(h8, vh), acc[(BLK * 2) * 4 + B], 0, 0, 0);             \
        acc[(BLK * 2 + 1) * 4 + B] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[2 * BLK + 1], __builtin_bit_cast(h8, vl), acc[(BLK * 2 + 1) * 4 + B], 0, 0, 0); \
    }
    SMH_MK_BYTE(u0, 0, 0)
    SMH_MK_BYTE(u0, 0, 1)
    SMH_MK_BYTE(u0, 0, 2)
    SMH_MK_BYTE(u0, 0, 3)
    SMH_MK_BYTE(u1, 1, 0)
    SMH_MK_BYTE(u1, 1, 1)
    SMH_MK_BYTE(u1, 1, 2)
    SMH_MK_BYTE(u1, 1, 3)
#undef SMH_MK_BYTE
}

// ---- folding the stream waves' accumulators through LDS ---------------------------------------------------
// image of a wave's 16 tiles: lane-major, 16 f4 per lane with a pitch of 17 f4 (conflict-free 128-bit
// accesses, tile offsets are immediates); only the lanes that hold rows < 4*mr take part
constexpr int MK_IMG_PITCH = 68;                     // floats per lane
__device__ __forceinline__ void img_store(float *img, int lanes_in, int lane, const f4 (&val)[16]) {
    if (lane < lanes_in) {
        float *mine = img + lane * MK_IMG_PITCH;
#pragma unroll
        for (int t = 0; t < 16; ++t) *reinterpret_cast<f4 *>(mine + 4 * t) = val[t];
    }
}
// val += image when `take` (wave-uniform); without control flow, so the accumulators stay in place
__device__ __forceinline__ void img_add(const float *img, int lanes_in, int lane, bool take, f4 (&val)[16]) {
    const float *mine = img + min(lane, lanes_in - 1) * MK_IMG_PITCH;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        const f4 v = *reinterpret_cast<const f4 *>(mine + 4 * t);
#pragma unroll
        for (int r = 0; r < 4; ++r) val[t][r] += take ? v[r] : 0.f;
    }
}
// Two rounds fold the four stream waves: waves 2,3 -> waves 0,1, then wave 1 -> wave 0, which leaves the
// image of the sum in slot 0.  The control waves run wg_fold_barriers, which has the same barriers.
__device__ __forceinline__ void wg_fold(f4 (&val)[16], float *red, int mr, int wave, int lane) {
    static_assert(MK_STREAM_WAVES == 4, "the fold is written for four stream waves");
    const int lanes_in = 16 * mr, slot = lanes_in * MK_IMG_PITCH;
    if (wave >= 2) img_store(red + (wave - 2) * slot, lanes_in, lane, val);
    wg_sync();
    img_add(red + (wave & 1) * slot, lanes_in, lane, wave < 2, val);
    wg_sync();
    if (wave == 1) img_store(red, lanes_in, lane, val);
    wg_sync();
    img_add(red, lanes_in, lane, wave == 0, val);
    wg_sync();
    if (wave == 0) img_store(red, lanes_in, lane, val);
    wg_sync();
}
__device__ __forceinline__ void wg_fold_barriers() {
#pragma unroll
    for (int i = 0; i < 5; ++i) wg_sync();
}

// ---- control side: activations of the phase into LDS ------------------------------------------------------
// x tile of step j: [M][32] halves at xbuf + j*M*64.  Steps j < nA are steps kA0.. of the first unit,
// the others steps 0.. of the next unit.
__device__ __forceinline__ void load_x(CParams &p, CLayer &L, int ph, uint8_t *xbuf, int n, int nA, int kA0,
                                       int ctid, int lane) {
    const int M = p.M;
    const int per_step = 4 * M;                       // 16-byte chunks per step
    const int steps_per_pass = (MK_CONTROL_WAVES * 64) / per_step;
    const int jj = ctid / per_step, rem = ctid - jj * per_step;
    const int m = rem >> 2, ch = rem & 3;
    const bool norm = (ph == MK_QKV || ph == MK_W13);
    float rstd = 0.f;
    if (norm) {
        // lane 16q + m adds every fourth unit's sum of squares of row m (loads issued together), the four
        // quarters are added across the wave, and lane m ends up with the row's 1/rms
        const float *ss = p.ssq + (long)(ph == MK_QKV ? 1 : 0) * (p.dim / 256) * M;
        const int units = p.dim / 256, mm = lane & 15, qq = lane >> 4;
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int u = qq + 4 * i;
            v[i] = (mm < M && u < units) ? ld_f32(ss + (long)u * M + mm) : 0.f;
        }
        float tot = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) tot += v[i];
        tot += __shfl_xor(tot, 16, 64);
        tot += __shfl_xor(tot, 32, 64);
        const float r = rms_factor(tot, p.dim, p.eps);
        rstd = __shfl(r, m, 64);
    }
    const half_t *src;
    long ld;
    const half_t *wn = nullptr;
    if (ph == MK_QKV) { src = p.h; ld = p.dim; wn = L.attn_norm; }
    else if (ph == MK_O) { src = p.attn_out; ld = (long)p.H * 128; }
    else if (ph == MK_W13) { src = p.h; ld = p.dim; wn = L.ffn_norm; }
    else { src = p.act; ld = p.ffn; }
    if (jj >= steps_per_pass) return;
    for (int j = jj; j < n; j += steps_per_pass) {
        const int kstep = j < nA ? kA0 + j : j - nA;
        const long k = (long)kstep * 32 + ch * 8;
        const half_t *sp = src + (long)m * ld + k;
        const u32x2 lo = ld_u64(sp), hi = ld_u64(sp + 4);
        h8 v = __builtin_bit_cast(h8, u32x4{lo[0], lo[1], hi[0], hi[1]});
        if (norm) {
            const h8 wv = *reinterpret_cast<const h8 *>(wn + k);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const half_t nv = scale_to_half(v[i], rstd);
                v[i] = nv * wv[i];
            }
        }
        *reinterpret_cast<h8 *>(xbuf + ((long)j * M + m) * 64 + ch * 16) = v;
    }
}

// sum of the partials of unit `u` for row m, columns col..col+3 (workgroup order)
struct UnitSource {
    int first, last, first_slot;
};
__device__ __forceinline__ UnitSource unit_source(const MegaMatrix &g, int u) {
    UnitSource s;
    unit_contributors(g, u, s.first, s.last);
    int a, b;
    wg_range(g, s.first, a, b);
    s.first_slot = (a < u * g.steps) ? 1 : 0;     // only the first contributor can have begun in the previous unit
    return s;
}
__device__ __forceinline__ f4 unit_sum4(CParams &p, const UnitSource &s, int m, int col) {
    f4 tot = {0.f, 0.f, 0.f, 0.f};
    for (int w = s.first; w <= s.last; w += 4) {
        f4 v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int ww = w + i;
            const int slot = (ww == s.first) ? s.first_slot : 0;
            v[i] = (ww <= s.last) ? ld_f4(p.slabs + (((long)ww * 2 + slot) * p.M + m) * 256 + col) : f4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) tot += v[i];
    }
    return tot;
}
__device__ __forceinline__ float unit_sum1(CParams &p, const UnitSource &s, int m, int col) {
    float tot = 0.f;
    for (int w = s.first; w <= s.last; w += 4) {
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int ww = w + i;
            const int slot = (ww == s.first) ? s.first_slot : 0;
            v[i] = (ww <= s.last) ? ld_f32(p.slabs + (((long)ww * 2 + slot) * p.M + m) * 256 + col) : 0.f;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) tot += v[i];
    }
    return tot;
}
// two fp16 values of adjacent lanes as one coherent 4-byte store (even lanes store)
__device__ __forceinline__ void st_half_pairs(half_t *row, int lane, half_t v) {
    const uint32_t mine = __builtin_bit_cast(uint16_t, v);
    const uint32_t next = (uint32_t)__shfl_down((int)mine, 1, 64);
    if ((lane & 1) == 0) st_u32(row + lane, mine | (next << 16));
}

// ---- finishers: one control wave completes row m of a unit ---------------------------------------------------
__device__ __forceinline__ void finish_residual(CParams &p, const MegaMatrix &g, int u, int m, int lane, int parity) {
    const UnitSource s = unit_source(g, u);
    const f4 acc = unit_sum4(p, s, m, 4 * lane);
    half_t *hp = p.h + (long)m * p.dim + (long)u * 256 + 4 * lane;
    const h4 r = ld_h4(hp);
    h4 o;
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const half_t v = (half_t)acc[j];
        o[j] = (half_t)((float)r[j] + (float)v);
        ss += (float)o[j] * (float)o[j];
    }
    st_h4(hp, o);
    ss = wave_sum(ss);
    if (lane == 0) st_f32(p.ssq + ((long)parity * (p.dim / 256) + u) * p.M + m, ss);
}
__device__ __forceinline__ void finish_qkv(CParams &p, CLayer &L, const MegaMatrix &g, int u, int m, int lane) {
    const UnitSource s = unit_source(g, u);
    int sg = 0;
    if (u >= g.unit0[1]) sg = 1;
    if (u >= g.unit0[2]) sg = 2;
    const int t = *p.t_dev, pos = *p.pos_dev;
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
        const int head = (u - pick3(g.unit0, sg)) * 2 + hh;
        half_t x1 = (half_t)unit_sum1(p, s, m, hh * 128 + lane);
        half_t x2 = (half_t)unit_sum1(p, s, m, hh * 128 + 64 + lane);
        if (sg == 2) {
            half_t *pv = p.cur_v + ((long)m * p.Hkv + head) * 128;
            st_half_pairs(pv, lane, x1);
            st_half_pairs(pv + 64, lane, x2);
            if (t >= 0 && t < p.Smax) {
                const long row = ((long)m * p.Smax + t) * p.Hkv + head;
                kv_store_row2(x1, x2, L.cache_v + row * 64, L.cache_vs + row * 2, lane);
            }
            continue;
        }
        rope_pair2(x1, x2, p.cos_tab[(long)pos * 64 + lane], p.sin_tab[(long)pos * 64 + lane]);
        if (sg == 0) {
            half_t *pq = p.q + ((long)m * p.H + head) * 128;
            st_half_pairs(pq, lane, x1);
            st_half_pairs(pq + 64, lane, x2);
        } else {
            half_t *pk = p.cur_k + ((long)m * p.Hkv + head) * 128;
            st_half_pairs(pk, lane, x1);
            st_half_pairs(pk + 64, lane, x2);
            if (t >= 0 && t < p.Smax) {
                const long row = ((long)m * p.Smax + t) * p.Hkv + head;
                kv_store_row2(x1, x2, L.cache_k + row * 64, L.cache_ks + row * 2, lane);
            }
        }
    }
}
__device__ __forceinline__ void finish_silu(CParams &p, const MegaMatrix &g, int pair, int m, int lane) {
    const UnitSource sg = unit_source(g, pair), su = unit_source(g, g.unit0[1] + pair);
    const f4 ga = unit_sum4(p, sg, m, 4 * lane), ua = unit_sum4(p, su, m, 4 * lane);
    h4 o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float gf = (float)(half_t)ga[j];
        const half_t sl = (half_t)(gf / (1.0f + expf(-gf)));
        o[j] = sl * (half_t)ua[j];
    }
    st_h4(p.act + (long)m * p.ffn + (long)pair * 256 + 4 * lane, o);
}

// control wave cw publishes rows m = cw, cw+4, .. of the workgroup's partial of unit u and finishes them if last
__device__ __forceinline__ void control_unit(CParams &p, CLayer &L, int ph, int u, int slot, int w, int cw,
                                             int lane, f4 (&rows)[4]) {
    const MegaMatrix g = matrix_of(p, ph);
    const int M = p.M;
    // rows were read from the LDS image by the caller (before the barrier that frees it)
#pragma unroll
    for (int gi = 0; gi < 4; ++gi) {         // constant register indices: rows[] must not be indexed at run time
        const int m = 4 * gi + cw;
        if (m < M) st_f4(p.slabs + (((long)w * 2 + slot) * M + m) * 256 + 4 * lane, rows[gi]);
    }
    if (cw >= M) return;                     // this wave owns no row
    wait_vmem();
    // arrival: the counter belongs to (phase, unit or pair, control wave)
    int cu = u, expected;
    {
        int f, l;
        unit_contributors(g, u, f, l);
        expected = l - f + 1;
        if (ph == MK_W13) {
            const int half = g.unit0[1];
            cu = u >= half ? u - half : u;
            int f2, l2;
            unit_contributors(g, u >= half ? u - half : u + half, f2, l2);
            expected += l2 - f2 + 1;
        }
    }
    uint32_t *cnt = p.unit_cnt + ((long)ph * p.max_units + cu) * MK_CONTROL_WAVES + cw;
    uint32_t prev = 0;
    if (lane == 0) prev = __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    prev = (uint32_t)__builtin_amdgcn_readfirstlane((int)prev);
    if (prev != (uint32_t)expected - 1u) return;
    if (lane == 0) st_u32(cnt, 0u);
    for (int m = cw; m < M; m += 4) {
        if (ph == MK_QKV) finish_qkv(p, L, g, u, m, lane);
        else if (ph == MK_O) finish_residual(p, g, u, m, lane, 0);
        else if (ph == MK_W13) finish_silu(p, g, cu, m, lane);
        else finish_residual(p, g, u, m, lane, 1);
    }
}

// ---- attention items ------------------------------------------------------------------------------------------
__device__ __forceinline__ RowRegs row_from_pairs(u32x2 lo, u32x2 hi) {
    RowRegs r;
    r.a02 = as_h2(pack_lo16(lo[0], lo[1]));
    r.a13 = as_h2(pack_hi16(lo[0], lo[1]));
    r.b02 = as_h2(pack_lo16(hi[0], hi[1]));
    r.b13 = as_h2(pack_hi16(hi[0], hi[1]));
    return r;
}
__device__ __forceinline__ void soft_init(SoftState &st) {
    st.m = -INFINITY;
    st.l = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) st.o[j] = 0.f;
}
// merge the four 16-lane groups of a wave; afterwards every lane holds the wave's state for its dims
__device__ __forceinline__ void soft_merge_groups(SoftState &st) {
#pragma unroll
    for (int sh = 16; sh <= 32; sh <<= 1) {
        const float m2 = __shfl_xor(st.m, sh, 64);
        const float l2 = __shfl_xor(st.l, sh, 64);
        float o2[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) o2[j] = __shfl_xor(st.o[j], sh, 64);
        soft_merge(st, m2, l2, o2);
    }
}
// partial record: o[128] in dimension order, m at [128], l at [129]
__device__ __forceinline__ void part_store_lds(float *rec, int c, const SoftState &st) {
    *reinterpret_cast<f4 *>(rec + 4 * c) = f4{st.o[0], st.o[2], st.o[1], st.o[3]};
    *reinterpret_cast<f4 *>(rec + 64 + 4 * c) = f4{st.o[4], st.o[6], st.o[5], st.o[7]};
    if (c == 0) {
        rec[128] = st.m;
        rec[129] = st.l;
    }
}
__device__ __forceinline__ void part_merge_lds(SoftState &st, const float *rec, int c) {
    const f4 lo = *reinterpret_cast<const f4 *>(rec + 4 * c), hi = *reinterpret_cast<const f4 *>(rec + 64 + 4 * c);
    const float o2[8] = {lo[0], lo[2], lo[1], lo[3], hi[0], hi[2], hi[1], hi[3]};
    soft_merge(st, rec[128], rec[129], o2);
}
__device__ __forceinline__ void part_merge_global(SoftState &st, const float *rec, int c) {
    const f4 lo = ld_f4(rec + 4 * c), hi = ld_f4(rec + 64 + 4 * c);
    typedef float f2 __attribute__((ext_vector_type(2)));
    const f2 ml = __builtin_bit_cast(f2, ld_u64(rec + 128));
    const float o2[8] = {lo[0], lo[2], lo[1], lo[3], hi[0], hi[2], hi[1], hi[3]};
    soft_merge(st, ml[0], ml[1], o2);
}

// One item = (head, prefix chunk) or (head, suffix), executed by the stream waves; it has four
// workgroup barriers, which the control waves execute as well.
__device__ __forceinline__ void attention_item(CParams &p, CLayer &L, int item, float *part, uint32_t *flag,
                                               int wave, int lane) {
    const int per_head = p.chunks + 1;
    const int h = item / per_head, ck = item - h * per_head;
    const int c = lane & 15, g = lane >> 4;
    const int M = p.M;
    {
        for (int b = 0; b < M; ++b) {
            const half_t *qp = p.q + ((long)b * p.H + h) * 128;
            const RowRegs qr = row_from_pairs(ld_u64(qp + 4 * c), ld_u64(qp + 64 + 4 * c));
            SoftState st;
            soft_init(st);
            if (ck < p.chunks) {
                const int r0 = ck * p.att_rows, r1 = min(r0 + p.att_rows, p.P);
#pragma unroll 4
                for (int rq = r0 + 4 * wave; rq < r1; rq += 4 * MK_STREAM_WAVES) {
                    const int r = rq + g;
                    if (r < r1) {
                        const long off = ((long)r * p.Hkv + h) * 128;
                        const RowRegs kr = row_from_fp16(L.prefix_k + off, c);
                        const RowRegs vr = row_from_fp16(L.prefix_v + off, c);
                        soft_add_row(st, row_dot(kr, qr) * p.scale_log2, vr);
                    }
                }
            } else {
                const int len = min(*p.t_dev, p.Smax);
                for (int t = 4 * wave + g; t < len; t += 4 * MK_STREAM_WAVES) {
                    const long row = ((long)b * p.Smax + t) * p.Hkv + h;
                    const uint32_t kb = *reinterpret_cast<const uint32_t *>(L.cache_k + row * 64 + 4 * c);
                    const uint32_t vb = *reinterpret_cast<const uint32_t *>(L.cache_v + row * 64 + 4 * c);
                    const uint32_t ksc = *reinterpret_cast<const uint32_t *>(L.cache_ks + row * 2);
                    const uint32_t vsc = *reinterpret_cast<const uint32_t *>(L.cache_vs + row * 2);
                    soft_add_row(st, row_dot(row_from_q40(kb, ksc), qr) * p.scale_log2, row_from_q40(vb, vsc));
                }
                if (wave == 0 && g == 0) {         // the new token's exact K/V
                    const long off = ((long)b * p.Hkv + h) * 128;
                    const RowRegs kr = row_from_pairs(ld_u64(p.cur_k + off + 4 * c), ld_u64(p.cur_k + off + 64 + 4 * c));
                    const RowRegs vr = row_from_pairs(ld_u64(p.cur_v + off + 4 * c), ld_u64(p.cur_v + off + 64 + 4 * c));
                    soft_add_row(st, row_dot(kr, qr) * p.scale_log2, vr);
                }
            }
            soft_merge_groups(st);
            if (g == 0) part_store_lds(part + ((long)wave * M + b) * MK_PART, c, st);
        }
    }
    wg_sync();
    {
        // wave v folds the stream waves' partials of branches v, v+4, .. and publishes the workgroup's partial
        for (int b = wave; b < M; b += MK_STREAM_WAVES) {
            SoftState st;
            soft_init(st);
            for (int wv = g; wv < MK_STREAM_WAVES; wv += 4) part_merge_lds(st, part + ((long)wv * M + b) * MK_PART, c);
            soft_merge_groups(st);
            if (g == 0) {
                float *rec = p.att_part + ((long)item * M + b) * MK_PART;
                st_f4(rec + 4 * c, f4{st.o[0], st.o[2], st.o[1], st.o[3]});
                st_f4(rec + 64 + 4 * c, f4{st.o[4], st.o[6], st.o[5], st.o[7]});
                if (c == 0) st_u64(rec + 128, u32x2{__builtin_bit_cast(uint32_t, st.m), __builtin_bit_cast(uint32_t, st.l)});
            }
        }
        wait_vmem();
    }
    wg_sync();
    if (wave == 0 && lane == 0) {
        const uint32_t prev = __hip_atomic_fetch_add(p.att_cnt + h, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const bool last = prev == (uint32_t)per_head - 1u;
        if (last) st_u32(p.att_cnt + h, 0u);
        *flag = last ? 1u : 0u;
    }
    wg_sync();
    if (*flag != 0u) {
        for (int b = wave; b < M; b += MK_STREAM_WAVES) {
            SoftState st;
            soft_init(st);
            for (int i = g; i < per_head; i += 4) part_merge_global(st, p.att_part + ((long)(h * per_head + i) * M + b) * MK_PART, c);
            soft_merge_groups(st);
            if (g == 0) {
                const float inv = st.l > 0.f ? 1.0f / st.l : 0.f;
                half_t *op = p.attn_out + ((long)b * p.H + h) * 128;
                st_h4(op + 4 * c, h4{(half_t)(st.o[0] * inv), (half_t)(st.o[2] * inv), (half_t)(st.o[1] * inv), (half_t)(st.o[3] * inv)});
                st_h4(op + 64 + 4 * c, h4{(half_t)(st.o[4] * inv), (half_t)(st.o[6] * inv), (half_t)(st.o[5] * inv), (half_t)(st.o[7] * inv)});
            }
        }
        wait_vmem();
    }
    wg_sync();
}

// ---- the kernel -------------------------------------------------------------------------------------------------
// The two roles are separate straight pieces of code that execute the same sequence of workgroup
// barriers; the comments name the barriers so that the two sides can be matched.
struct PhaseWork {
    int n, nA, kA0, uA, n_units;
};
__device__ __forceinline__ PhaseWork phase_work(const MegaMatrix &gm, int w) {
    PhaseWork k;
    int a, b;
    wg_range(gm, w, a, b);
    k.n = b - a;
    k.uA = k.n > 0 ? (int)((uint32_t)a / (uint32_t)gm.steps) : 0;
    k.kA0 = a - k.uA * gm.steps;
    k.nA = min(k.n, gm.steps - k.kA0);
    k.n_units = k.n == 0 ? 0 : (k.n > k.nA ? 2 : 1);
    return k;
}
__device__ __forceinline__ int matrix_phase(int phase) { return phase == 0 ? MK_QKV : phase == 2 ? MK_O : phase == 3 ? MK_W13 : MK_W2; }
__device__ __forceinline__ int launder(int v) {
    asm volatile("" : "+v"(v));
    return v;
}

__device__ __forceinline__ void stream_role(CParams &p, uint8_t *lds, int w, int wave, int lane0) {
    uint8_t *xbuf = lds + p.xbuf_off;
    float *red = reinterpret_cast<float *>(lds + p.red_off);
    uint32_t *flag = reinterpret_cast<uint32_t *>(lds + p.flag_off);
    const int M = p.M;
    DecodeConsts C{0x00F000F0u, 0x000F000Fu, 0x54005400u, 0x64006400u};
    asm volatile("" : "+s"(C.mask_hi), "+s"(C.mask_lo));
    asm volatile("" : "+v"(C.magic_hi), "+v"(C.magic_lo));
    Cursor cur{};
    Ring ring{};
    cursor_enter(cur, p, w, wave, lane0);
    ring.base = (uint32_t)(wave * (p.stages * MK_STAGE));
    ring.stages = p.stages;
    ring_fill(ring, cur, p, lds, w, wave, lane0);
    wg_sync();                                                   // [init]
#ifdef SMH_MEGA_DEBUG
    const bool trace_on = wave == 0 && (w == 0 || w == 131);
    const int trace_slot = w == 0 ? 0 : 1;
    int trace_i = 0;
#endif
    MTR(trace_slot, 1);

    for (int layer = 0; layer < p.n_layers; ++layer) {
        CLayer &L = layer_of(p, layer);
        for (int phase = 0; phase < 5; ++phase) {
            // lane-dependent addresses are formed again in every phase: hoisted out of the layer loop
            // they would be hundreds of live registers
            const int lane = launder(lane0);
            const int c = lane & 15, g = lane >> 4;
            if (phase == 1) {
                wg_sync();                                           // [att] inputs are visible
                MTR(trace_slot, 10);
                const int items = p.H * (p.chunks + 1);
                for (int item = w; item < items; item += p.G) attention_item(p, L, item, reinterpret_cast<float *>(xbuf), flag, wave, lane);
                MTR(trace_slot, 11);
                continue;
            }
            const int ph = matrix_phase(phase);
            const PhaseWork k = phase_work(matrix_of(p, ph), w);
            wg_sync();                                               // [x] activations are in LDS
            MTR(trace_slot, 20 + phase);
            int j = wave;
            for (int ui = 0; ui < k.n_units; ++ui) {
                const int j_end = ui == 0 ? k.nA : k.n;
                f4 val[16], corr[4];
#pragma unroll
                for (int t = 0; t < 16; ++t) val[t] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int t = 0; t < 4; ++t) corr[t] = f4{0.f, 0.f, 0.f, 0.f};
                const int row = min(c, M - 1);
                for (; j < j_end; j += MK_STREAM_WAVES) {
                    ring_wait_head(ring);
                    step_consume(lds + ring.base + ring.head * MK_STAGE, xbuf + (long)j * M * 64, c, g, row, C, val, corr);
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");            // the stage has been read
                    ring.head = uni((ring.head + 1 == ring.stages) ? 0 : ring.head + 1);
                    ring.inflight = uni(ring.inflight - 1);
                    ring_fill(ring, cur, p, lds, w, wave, lane);
                }
                // take the nibble offsets out: tiles of the high nibbles carry 72, of the low nibbles 1032
#pragma unroll
                for (int t = 0; t < 16; ++t) {
                    const int bh = t >> 2;
                    val[t] -= ((bh & 1) ? 1032.f : 72.f) * corr[bh];
                }
                MTR(trace_slot, 30 + phase);
                wg_fold(val, red, p.mr, wave, lane);           // [fold rounds] ... [sum ready]
                wg_sync();                                           // [sum taken] the image may be overwritten
                MTR(trace_slot, 40 + phase);
            }
        }
    }
}

__device__ __forceinline__ void control_role(CParams &p, uint8_t *lds, int w, int cw, int lane0) {
    uint8_t *xbuf = lds + p.xbuf_off;
    const float *red = reinterpret_cast<const float *>(lds + p.red_off);
    const int M = p.M;
    uint32_t *words = reinterpret_cast<uint32_t *>(lds + p.flag_off);
    const uint32_t arrivals = (uint32_t)(p.G < MK_GROUPS ? p.G : MK_GROUPS);   // top-counter increments per grid barrier
    const uint32_t base = ld_u32(p.sync + 1);
    if (cw == 0 && lane0 == 0) {
        words[1] = 0u;
        words[2] = 0u;
    }
    wg_sync();                                                   // [init]
    uint32_t barrier_no = 0;

    // ---- embedding: unit u of the hidden state by workgroup u ----
    if (w < p.dim / 256) {
        for (int m = cw; m < M; m += MK_CONTROL_WAVES) {
            const long tok = p.tokens[m];
            const h4 v = *reinterpret_cast<const h4 *>(p.emb + tok * p.dim + (long)w * 256 + 4 * lane0);
            st_h4(p.h + (long)m * p.dim + (long)w * 256 + 4 * lane0, v);
            float ss = 0.f;
#pragma unroll
            for (int j = 0; j < 4; ++j) ss += (float)v[j] * (float)v[j];
            ss = wave_sum(ss);
            if (lane0 == 0) st_f32(p.ssq + ((long)(p.dim / 256) + w) * M + m, ss);
        }
    }
    grid_arrive(p, words, w, lane0);
#ifdef SMH_MEGA_DEBUG
    const bool trace_on = cw == 0 && (w == 0 || w == 131);
    const int trace_slot = w == 0 ? 2 : 3;
    int trace_i = 0;
#endif
    MTR(trace_slot, 1);

    for (int layer = 0; layer < p.n_layers; ++layer) {
        CLayer &L = layer_of(p, layer);
        for (int phase = 0; phase < 5; ++phase) {
            const int lane = launder(lane0);
            ++barrier_no;
            MTR(trace_slot, 50 + phase);
            grid_wait(p, words, cw, base + barrier_no * arrivals, barrier_no);
            MTR(trace_slot, 60 + phase);
            if (phase == 1) {
                wg_sync();                                           // [att]
                const int items = p.H * (p.chunks + 1);
                for (int item = w; item < items; item += p.G) {
                    wg_sync();
                    wg_sync();
                    wg_sync();
                    wg_sync();
                }
                grid_arrive(p, words, w, lane);
                continue;
            }
            const int ph = matrix_phase(phase);
            const PhaseWork k = phase_work(matrix_of(p, ph), w);
            if (k.n > 0) load_x(p, L, ph, xbuf, k.n, k.nA, k.kA0, cw * 64 + lane, lane);
            MTR(trace_slot, 70 + phase);
            wg_sync();                                               // [x]
            for (int ui = 0; ui < k.n_units; ++ui) {
                wg_fold_barriers();                              // [fold rounds] ... [sum ready]
                // control wave cw takes its rows (r = cw) out of the image before the image is reused
                f4 rows[4];
                const int blk = lane >> 5, hf = (lane >> 4) & 1, cc = lane & 15;
#pragma unroll
                for (int gi = 0; gi < 4; ++gi) {
                    rows[gi] = f4{0.f, 0.f, 0.f, 0.f};
                    if (gi < p.mr) {
#pragma unroll
                        for (int bb = 0; bb < 4; ++bb) {
                            const int t = (blk * 2 + hf) * 4 + bb;
                            rows[gi][bb] = red[(gi * 16 + cc) * MK_IMG_PITCH + 4 * t + cw];
                        }
                    }
                }
                wg_sync();                                           // [sum taken]
                MTR(trace_slot, 80 + phase);
                control_unit(p, L, ph, k.uA + ui, ui, w, cw, lane, rows);
                MTR(trace_slot, 90 + phase);
            }
            grid_arrive(p, words, w, lane);
            MTR(trace_slot, 100 + phase);
        }
    }
    ++barrier_no;
    grid_wait(p, words, cw, base + barrier_no * arrivals, barrier_no);
    if (w == 0 && cw == 0 && lane0 == 0) st_u32(p.sync + 1, base + barrier_no * arrivals);
    wait_vmem();
}

__global__ __launch_bounds__(MK_THREADS) void decode_mega_kernel(const MegaParams *params) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    CParams &p = *reinterpret_cast<CParams *>(reinterpret_cast<uintptr_t>(params));
    // workgroups are dealt round-robin to the 8 XCDs; consecutive LOGICAL workgroups (which stream adjacent
    // column units and share the cache lines of their scales) are placed behind the same L2
    int w = uni((int)blockIdx.x);
    if ((p.G & 7) == 0) w = uni((w & 7) * (p.G >> 3) + (w >> 3));
    const int wave = uni((int)threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (wave < MK_STREAM_WAVES) stream_role(p, lds, w, wave, lane);
    else control_role(p, lds, w, wave - MK_STREAM_WAVES, lane);
}

}  // namespace smh

using namespace smh;

// ---- host side -----------------------------------------------------------------------------------------------------
namespace {

struct MegaPlan {
    MegaParams p;
    size_t lds_bytes;
    size_t off_params, off_q, off_k, off_v, off_attn, off_act, off_slabs, off_ssq, off_part, off_ucnt, off_acnt, off_sync, total;
};

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

int mega_plan(MegaPlan &pl, int n_layers, int M, int dim, int H, int Hkv, int ffn, int P, int Smax, int G, const char *who) {
    SMH_REQUIRE(M >= 1 && M <= MK_MAX_M, "%s: M=%d outside [1,%d]", who, M, MK_MAX_M);
    SMH_REQUIRE(H == Hkv, "%s: H=%d Hkv=%d (this kernel covers multi-head attention; grouped heads use the operator kernels)", who, H, Hkv);
    SMH_REQUIRE(dim % 256 == 0 && ffn % 256 == 0 && (H * 128) % 256 == 0 && dim > 0 && dim <= 8192 && ffn > 0,
                "%s: dim=%d ffn=%d H=%d (dim, ffn and 128*H must be multiples of 256)", who, dim, ffn, H);
    SMH_REQUIRE(n_layers >= 1 && P >= 0 && Smax >= 1 && G >= 1, "%s: n_layers=%d P=%d Smax=%d G=%d", who, n_layers, P, Smax, G);
    MegaParams &p = pl.p;
    p = MegaParams{};
    p.n_layers = n_layers; p.M = M; p.dim = dim; p.H = H; p.Hkv = Hkv; p.ffn = ffn; p.P = P; p.Smax = Smax; p.G = G;
    // attention items per head: prefix chunks + the suffix; sized so that one round of workgroups covers them
    {
        int want = G / H - 1;
        if (want < 1) want = 1;
        int rows = ((P + want - 1) / want + 15) / 16 * 16;
        if (rows < 16) rows = 16;
        p.att_rows = rows;
        p.chunks = (P + rows - 1) / rows;
    }
    auto set = [&](int ph, int nseg, const int *ids, const int *ns, int K) {
        MegaMatrix &g = p.mat[ph];
        g.nseg = nseg;
        int u0 = 0;
        for (int i = 0; i < nseg; ++i) {
            g.seg_id[i] = ids[i];
            g.seg_n[i] = ns[i];
            g.unit0[i] = u0;
            u0 += ns[i] / 256;
        }
        g.K = K;
        g.steps = K / 32;
        g.units = u0;
        g.T = g.units * g.steps;
        g.geff = g.T < G ? g.T : G;
    };
    const int qkv_ids[3] = {0, 1, 2}, qkv_n[3] = {H * 128, Hkv * 128, Hkv * 128};
    const int o_ids[1] = {3}, o_n[1] = {dim};
    const int w13_ids[2] = {4, 5}, w13_n[2] = {ffn, ffn};
    const int w2_ids[1] = {6}, w2_n[1] = {dim};
    set(MK_QKV, 3, qkv_ids, qkv_n, dim);
    set(MK_O, 1, o_ids, o_n, H * 128);
    set(MK_W13, 2, w13_ids, w13_n, dim);
    set(MK_W2, 1, w2_ids, w2_n, ffn);
    int n_max = 1;
    p.max_units = 1;
    for (int ph = 0; ph < MK_MATRIX_PHASES; ++ph) {
        const MegaMatrix &g = p.mat[ph];
        SMH_REQUIRE(g.K % 32 == 0 && g.units <= g.geff, "%s: matrix phase %d: K=%d units=%d over %d workgroups", who, ph, g.K, g.units, g.geff);
        SMH_REQUIRE((long)g.T * (G + 1) < (1L << 31), "%s: matrix phase %d too large", who, ph);
        const int per = (g.T + g.geff - 1) / g.geff;
        if (per > n_max) n_max = per;
        if (g.units > p.max_units) p.max_units = g.units;
    }
    p.mr = (M + 3) / 4;
    const int x_bytes = (int)align_up((size_t)n_max * M * 64, 16);
    const int red_bytes = 2 * p.mr * 16 * MK_IMG_PITCH * 4;
    const int att_bytes = MK_STREAM_WAVES * M * MK_PART * 4;
    int scratch = x_bytes + red_bytes;
    if (att_bytes > scratch) scratch = att_bytes;
    p.stages = 0;
    for (int s = MK_MAX_STAGES; s >= 2; --s)
        if (MK_STREAM_WAVES * s * MK_STAGE + scratch + 64 <= MK_LDS_LIMIT) { p.stages = s; break; }
    SMH_REQUIRE(p.stages >= 2, "%s: LDS does not fit (scratch %d bytes)", who, scratch);
    static const int stage_cap = env_int("SMH_MEGA_STAGES", MK_MAX_STAGES);
    if (p.stages > stage_cap && stage_cap >= 2) p.stages = stage_cap;
    p.xbuf_off = MK_STREAM_WAVES * p.stages * MK_STAGE;
    p.red_off = p.xbuf_off + x_bytes;
    p.flag_off = p.xbuf_off + scratch;
    pl.lds_bytes = (size_t)p.flag_off + 64;
    p.spin_limit = 1 << 22;
    size_t o = 0;
    auto take = [&](size_t bytes) { size_t at = o; o = align_up(o + bytes, 256); return at; };
    pl.off_sync = take(MK_SYNC_BYTES);   // status words and barrier counters come first, then the parameter block
    pl.off_params = take(sizeof(MegaParams));
    pl.off_q = take((size_t)M * H * 128 * 2);
    pl.off_k = take((size_t)M * Hkv * 128 * 2);
    pl.off_v = take((size_t)M * Hkv * 128 * 2);
    pl.off_attn = take((size_t)M * H * 128 * 2);
    pl.off_act = take((size_t)M * ffn * 2);
    pl.off_slabs = take((size_t)G * 2 * M * 256 * 4);
    pl.off_ssq = take((size_t)2 * (dim / 256) * M * 4);
    pl.off_part = take((size_t)H * (p.chunks + 1) * M * MK_PART * 4);
    pl.off_ucnt = take((size_t)MK_MATRIX_PHASES * p.max_units * MK_CONTROL_WAVES * 4);
    pl.off_acnt = take((size_t)H * 4);
    pl.total = o;
    return 0;
}

}  // namespace

extern "C" size_t smh_decode_step_workspace_bytes(int n_layers, int M, int dim, int H, int Hkv, int ffn, int P, int Smax) {
    MegaPlan pl;
    if (mega_plan(pl, n_layers, M, dim, H, Hkv, ffn, P, Smax, 256, "smh_decode_step_workspace_bytes") != 0) return 0;
    return pl.total;
}

namespace {
struct Prepared {
    int G;
    size_t lds_bytes;
};
std::mutex g_prepared_mutex;
std::map<const void *, Prepared> g_prepared;          // keyed by workspace
}  // namespace

extern "C" int smh_decode_prepare(const smh_decode_layer *layers_dev, int n_layers, int M, int dim, int H, int Hkv, int ffn, int P,
                                  int Smax, float eps, const int64_t *tokens, const void *emb, const void *cos_tab,
                                  const void *sin_tab, const int32_t *pos_dev, const int32_t *t_dev, void *h_out, void *workspace,
                                  size_t workspace_bytes) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) {
        set_error("smh_decode_prepare: cannot query the device");
        return -1;
    }
    const int cus = prop.multiProcessorCount;
    const int G = cus < 256 ? cus : 256;
    MegaPlan pl;
    int st = mega_plan(pl, n_layers, M, dim, H, Hkv, ffn, P, Smax, G, "smh_decode_prepare");
    if (st) return st;
    SMH_REQUIRE(layers_dev && tokens && emb && cos_tab && sin_tab && pos_dev && t_dev && h_out && workspace, "smh_decode_prepare: null pointer");
    SMH_REQUIRE(workspace_bytes >= pl.total, "smh_decode_prepare: workspace %zu < %zu bytes", workspace_bytes, pl.total);
    SMH_REQUIRE(((uintptr_t)workspace & 255) == 0, "smh_decode_prepare: workspace must be 256-byte aligned");
    static_assert(sizeof(smh_decode_layer) == sizeof(MegaLayer), "layer descriptor layout");
    MegaParams &p = pl.p;
    uint8_t *ws = (uint8_t *)workspace;
    p.layers = reinterpret_cast<const MegaLayer *>(layers_dev);
    p.tokens = tokens;
    p.emb = (const half_t *)emb;
    p.cos_tab = (const half_t *)cos_tab;
    p.sin_tab = (const half_t *)sin_tab;
    p.pos_dev = pos_dev;
    p.t_dev = t_dev;
    p.h = (half_t *)h_out;
    p.q = (half_t *)(ws + pl.off_q);
    p.cur_k = (half_t *)(ws + pl.off_k);
    p.cur_v = (half_t *)(ws + pl.off_v);
    p.attn_out = (half_t *)(ws + pl.off_attn);
    p.act = (half_t *)(ws + pl.off_act);
    p.slabs = (float *)(ws + pl.off_slabs);
    p.ssq = (float *)(ws + pl.off_ssq);
    p.att_part = (float *)(ws + pl.off_part);
    p.unit_cnt = (uint32_t *)(ws + pl.off_ucnt);
    p.att_cnt = (uint32_t *)(ws + pl.off_acnt);
    p.sync = (uint32_t *)(ws + pl.off_sync);
    p.eps = eps;
    p.scale_log2 = 1.4426950408889634f / sqrtf(128.f);
    hipError_t e = hipDeviceSynchronize();                       // earlier steps may still use the workspace
    if (e == hipSuccess) e = hipMemset(workspace, 0, pl.total);
    if (e == hipSuccess) e = hipMemcpy(ws + pl.off_params, &p, sizeof(p), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipFuncSetAttribute((const void *)decode_mega_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, MK_LDS_LIMIT);
    if (e != hipSuccess) {
        set_error("smh_decode_prepare: %s", hipGetErrorString(e));
        return (int)e;
    }
    std::lock_guard<std::mutex> lock(g_prepared_mutex);
    g_prepared[workspace] = Prepared{G, pl.lds_bytes};
    return 0;
}

extern "C" int smh_decode_step(void *workspace, smh_stream_t stream) {
    Prepared pr;
    {
        std::lock_guard<std::mutex> lock(g_prepared_mutex);
        auto it = g_prepared.find(workspace);
        SMH_REQUIRE(it != g_prepared.end(), "smh_decode_step: workspace %p was not prepared (smh_decode_prepare)", workspace);
        pr = it->second;
    }
    const MegaParams *params = reinterpret_cast<const MegaParams *>((const uint8_t *)workspace + MK_SYNC_BYTES);
    hipLaunchKernelGGL(decode_mega_kernel, dim3((unsigned)pr.G), dim3(MK_THREADS), pr.lds_bytes, (hipStream_t)stream, params);
    return launch_status();
}

extern "C" int smh_decode_status(const void *workspace, uint32_t *status3) {
    SMH_REQUIRE(workspace && status3, "smh_decode_status: null pointer");
    hipError_t e = hipMemcpy(status3, workspace, 12, hipMemcpyDeviceToHost);
    if (e != hipSuccess) {
        set_error("smh_decode_status: %s", hipGetErrorString(e));
        return (int)e;
    }
    return 0;
}

#ifdef SMH_MEGA_DEBUG
// debugging aids of a -DSMH_MEGA_DEBUG build (not part of the ABI): byte offsets of q, cur_k, cur_v, attn_out, act,
// slabs, ssq, att_part inside the workspace, and the cycle trace
extern "C" int smhdbg_decode_offsets(int n_layers, int M, int dim, int H, int Hkv, int ffn, int P, int Smax, int G, size_t *out) {
    MegaPlan pl;
    if (mega_plan(pl, n_layers, M, dim, H, Hkv, ffn, P, Smax, G, "smhdbg_decode_offsets") != 0) return -1;
    out[0] = pl.off_q; out[1] = pl.off_k; out[2] = pl.off_v; out[3] = pl.off_attn; out[4] = pl.off_act;
    out[5] = pl.off_slabs; out[6] = pl.off_ssq; out[7] = pl.off_part;
    out[8] = pl.p.stages; out[9] = pl.lds_bytes;
    return 0;
}

extern "C" int smhdbg_read_trace(unsigned long long *out) {
    return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(smh_mega_trace), sizeof(unsigned long long) * 8 * 4096);
}
#endif
