/* smh.h - C ABI of the MI355X (gfx950) Q4_0 CodeLlama hot path.
 *
 * The reference (hongyihuang/spec-mcts) is pure Python + Triton and has no native boundary; each
 * entry point below replaces one Python-level operator or model method of the reference, cited
 * as file:line relative to the reference checkout.  A Python caller binds these with ctypes
 * (spec_mcts_amd/_lib.py does exactly that).
 *
 * Conventions
 *  - every pointer is a DEVICE pointer unless its name ends in _host;
 *  - fp16 data is IEEE binary16, row-major, innermost dimension contiguous;
 *  - Q4_0 data is the reference's layout (fp16_to_int4.py:52-96): 64-byte rows of packed signed
 *    nibbles, two 64-value groups per row (group 2p in the high nibbles, group 2p+1 in the low
 *    nibbles), one fp16 scale per group;  value = nibble * scale, nibble in [-8, 7];
 *  - a Q4_0 weight is the quantised TRANSPOSE of the [N,K] linear weight (fp16_to_int4.py:173):
 *    bytes viewed [K, N/2], scales viewed [K, N/64] (triton_kernels.py:481-482), N % 128 == 0;
 *  - kernels are enqueued on `stream` and never synchronise; nothing is allocated or freed;
 *  - return value: 0 on success, negative = invalid argument (see smh_last_error_string),
 *    positive = hipError_t from the launch.
 */
#ifndef SMH_H
#define SMH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *smh_stream_t; /* hipStream_t */

#define SMH_VERSION 1

/* epilogues of the Q4_0 matmul */
#define SMH_EPI_NONE 0     /* c = fp16(acc) */
#define SMH_EPI_RESIDUAL 1 /* c = fp16(residual + fp16(acc))   (h + wo(..), hf_model_q40_kv_shared.py:463-466) */

/* suffix KV formats of the decode attention */
#define SMH_KV_NONE 0
#define SMH_KV_FP16 1
#define SMH_KV_Q40 2

int smh_version(void);
/* message of the last failing call on the calling thread ("" if none) */
const char *smh_last_error_string(void);

/* ---- Q4_0 codec --------------------------------------------------------------------------
 * smh_q40_dequant replaces triton_deq_int40 / dequantize_q40 (triton_kernels.py:43-107):
 * rows 64-byte rows -> rows*128 fp16 values, bit-exact nibble*scale.
 * smh_q40_quantize replaces quantize_q40 (triton_kernels.py:12-41) for fp16 input with torch's
 * rounding: scale = fp16(absmax/7), code = rint(fp16(x/scale)), 0/0 -> 0. groups must be even. */
int smh_q40_dequant(const void *w, const void *s, void *out, long rows, smh_stream_t stream);
int smh_q40_quantize(const void *in, void *w, void *s, long groups, smh_stream_t stream);
/* smh_q40_quantize_f32: the same quantiser for checkpoint weights held in fp32 or bfloat16 (fp16_to_int4.py:169-184 runs
 * quantize_q40 on the checkpoint's own dtype; HF CodeLlama shards are bfloat16).  `in` holds the values widened to fp32;
 * src_bf16 != 0 says they were bfloat16.  torch's roundings for those types: scale = fp16(T(absmax / 7)) with T the source
 * type, code = rint(x / scale) with the quotient in fp32. */
int smh_q40_quantize_f32(const void *in, int src_bf16, void *w, void *s, long groups, smh_stream_t stream);

/* ---- Q4_0 matmul ---------------------------------------------------------------------------
 * c[M,N] = a[M,K] . deq(b_w, b_s)[K,N], fp16 operands, fp32 accumulation, one fp16 rounding;
 * replaces matmul_q40 (triton_kernels.py:471-500) = LinearQ4_0.forward
 * (hf_model_q40_kv_shared.py:228-236).  lda/ldc/ldr are row strides in elements.
 * Requires N % 128 == 0, K % 8 == 0, lda % 8 == 0, ldc % 4 == 0 and 16-byte aligned a.
 * smh_q40_matmul picks the GEMV kernel (M <= SMH_GEMV_MAX_M) or the LDS/MFMA GEMM.
 * workspace: smh_q40_matmul_workspace_bytes() bytes of scratch (no initialisation needed) that
 * holds the K-slice slabs between the producing kernel and the reduce kernel; calls that
 * overlap on different streams need separate workspaces. */
#define SMH_GEMV_MAX_M 16
size_t smh_q40_matmul_workspace_bytes(int max_m, int max_n);
int smh_q40_gemv(const void *a, int M, int K, long lda, const void *b_w, const void *b_s, int N,
                 void *c, long ldc, int epilogue, const void *residual, long ldr,
                 void *workspace, size_t workspace_bytes, smh_stream_t stream);
int smh_q40_gemm(const void *a, int M, int K, long lda, const void *b_w, const void *b_s, int N,
                 void *c, long ldc, int epilogue, const void *residual, long ldr,
                 void *workspace, size_t workspace_bytes, smh_stream_t stream);
int smh_q40_matmul(const void *a, int M, int K, long lda, const void *b_w, const void *b_s, int N,
                   void *c, long ldc, int epilogue, const void *residual, long ldr,
                   void *workspace, size_t workspace_bytes, smh_stream_t stream);

/* The block-of-32 flavour of Q4_0 that the benchmark's first configuration describes in words (32-weight blocks along the
 * input dimension, one fp16 scale = absmax / 8 per block, nibbles q in [0, 15], value = (q - 8) * scale).  The reference's
 * code has no such format (fp16_to_int4.py:52-96 is the 64-group, absmax / 7, signed-nibble layout above); these two entry
 * points exist so that that configuration can be run as written: smh_gq40_quantize packs fp16 values [blocks, 32] into
 * 16 bytes per block (element j in the low nibble of byte j, element j + 16 in the high nibble) + one fp16 scale, with the
 * reference quantiser's roundings (scale = fp16(absmax / 8), q = rint(fp16(x / scale)) + 8 cut to 0..15, 0 / 0 -> 8);
 * smh_gq40_dequant is its inverse, one fp16 multiply per weight.  Pointers 16-byte aligned. */
int smh_gq40_quantize(const void *in, void *packed, void *scale, long blocks, smh_stream_t stream);
int smh_gq40_dequant(const void *packed, const void *scale, void *out, long blocks, smh_stream_t stream);

/* ---- fused decode-layer operators ------------------------------------------------------------
 * The matmul kernels cut K into `ksplit` slices and leave one slab per slice,
 * partial[ksplit][M][n_total]; the operator that FOLLOWS the linear in the model adds the slabs
 * (in fp32, in slice order), rounds once to fp16 - the value matmul_q40 returns - and carries on, so no
 * kernel waits for another workgroup and a decode layer needs 4 weight-streaming launches.
 * The slabs hold fp32 at every batch size (a partial sum rounded to fp16 before the final addition is a cast point
 * the reference does not have); the consumer must be given the M (B for the rope operator) and the ksplit the
 * producer used.  Sizes below are in bytes.
 * Up to 3 weights that share the input (wq|wk|wv of Attention.forward,
 * hf_model_q40_kv_shared.py:313; w1|w3 of FeedForward.forward, :434) run as segments of one
 * launch; their outputs are concatenated along the columns (n_total = sum of n[i]).
 *
 * smh_q40_matmul_plan         ksplit the kernels will use for these dimensions on checkpoint-layout weights (depends on M, K, n only)
 * smh_q40_matmul_plan_tiled   the same for tiled weights (smh_q40_tile): equal up to 16 rows; above, tiled weights may take fewer slices
 * smh_q40_matmul_partial      produce the slabs; partial_bytes >= ksplit * M * n_total * 4
 * smh_partial_reduce          c[m][j] = fp16(sum) (+ residual) for columns col0 .. col0+N-1
 * smh_partial_rmsnorm         h_out = h_in + fp16(sum) (residual add of TransformerBlock.forward,
 *                             :463-466; h_in may be NULL), xn_out = RMSNorm(h_out) * weight (:129-134);
 *                             with partial == NULL it is a plain RMSNorm of h_in
 * smh_partial_silu_mul        slabs hold [w1 x | w3 x] (n_total = 2 * n_half): out = silu(.) * (.) (:434)
 * smh_partial_rope_append_kv  slabs hold [q | k | v] (n_total = (H + 2 Hkv) * D): rounds to fp16,
 *                             applies apply_rotary_emb (:173-203) to q and k at position *pos_dev,
 *                             writes q [B,H,D], k, v [B,Hkv,D] and appends Q4_0(k), Q4_0(v) to row
 *                             *t_dev of every branch's suffix cache (:365-371); cache_k may be NULL
 */
int smh_q40_matmul_plan(int M, int K, int nseg, const int *n);
int smh_q40_matmul_plan_tiled(int M, int K, int nseg, const int *n);
/* smh_q40_matmul_tiled_swiglu: out[M, n_half] = fp16(silu(fp16(a . gate))) * fp16(a . up) for tiled gate and up weights
 * [K, n_half] - `F.silu(self.w1(x)) * self.w3(x)` of FeedForward.forward (hf_model_q40_kv_shared.py:434) in ONE launch, with
 * the roundings of smh_q40_matmul_partial_tiled + smh_partial_silu_mul (every linear rounded to fp16 first) and no slab
 * in between.  17 <= M <= 128, K a multiple of 64, n_half a multiple of 128 and at most 16384 (all of K in one workgroup,
 * one workgroup per compute unit).  smh_q40_swiglu_fits: 1 when the shape is supported AND wide enough (n_half >= 8192) for
 * this to be the faster way; else use the two launches. */
int smh_q40_swiglu_fits(int M, int K, int n_half);
int smh_q40_matmul_tiled_swiglu(const void *a, int M, int K, long lda, const void *tiled_gate, const void *tiled_up, int n_half,
                                void *out, long ldo, smh_stream_t stream);
int smh_q40_matmul_partial(const void *a, int M, int K, long lda, int nseg, const void *const *w,
                           const void *const *s, const int *n, void *partial, size_t partial_bytes,
                           smh_stream_t stream);
/* Tiled weights.  The checkpoint layout written by fp16_to_int4.py:165-201 (bytes [K, N/2], scales [K, N/64])
 * is what every entry point above takes.  smh_q40_tile rewrites one weight, once, into the order the matmul
 * kernels consume it (256-column x 32-row tiles of 4352 contiguous bytes: nibbles in MFMA operand order, then the
 * tile's scales); smh_q40_matmul_partial_tiled is smh_q40_matmul_partial on such weights and leaves bit-identical
 * slabs - it replaces the same matmul_q40 (triton_kernels.py:471-500) calls, with fewer memory requests and fewer
 * decode instructions per weight.  tiled buffers: smh_q40_tiled_bytes(K, N) bytes, 128-byte aligned. */
size_t smh_q40_tiled_bytes(int K, int N);
int smh_q40_tile(const void *w, const void *s, int K, int N, void *tiled, size_t tiled_bytes, smh_stream_t stream);
int smh_q40_matmul_partial_tiled(const void *a, int M, int K, long lda, int nseg, const void *const *tiled,
                                 const int *n, void *partial, size_t partial_bytes, smh_stream_t stream);
/* smh_q40_matmul_partial_tiled_silu: w2(F.silu(w1 x) * w3 x) of FeedForward.forward (hf_model_q40_kv_shared.py:434) without
 * the launch between the two matmuls, for M <= 2 rows: the activations of the product are not read from memory but made by
 * every workgroup for its own K-slice from the gate|up slabs (columns 0..K-1 gate, K..2K-1 up, as smh_partial_silu_mul takes
 * them), with the same roundings; the slabs it leaves equal those of smh_partial_silu_mul + smh_q40_matmul_partial_tiled. */
int smh_q40_matmul_partial_tiled_silu(const void *gate_up_partial, int gate_up_ksplit, int M, int K, int nseg,
                                      const void *const *tiled, const int *n, void *partial, size_t partial_bytes,
                                      smh_stream_t stream);
/* RMSNorm.forward (hf_model_q40_kv_shared.py:85-94) of the residual stream followed by a linear, for up to 16 rows, as two
 * launches instead of three.  smh_partial_residual_sumsq is the first half of smh_partial_rmsnorm spread over 16
 * workgroups a row: h_out = h_in + fp16(sum of the slabs) and sums[m][0..15], partial sums of squares of h_out's row m
 * (fp32; added in index order they are smh_partial_rmsnorm's sum bit for bit).  smh_q40_matmul_partial_tiled_norm is
 * smh_q40_matmul_partial_tiled on a = RMSNorm(h) * norm_weight, which every workgroup makes for its own K-slice from h,
 * sums and norm_weight with smh_partial_rmsnorm's roundings; the slabs it leaves equal those of smh_partial_rmsnorm +
 * smh_q40_matmul_partial_tiled.  M rows x the K-slice must fit the workgroup's LDS: smh_q40_norm_in_fits says (1 / 0)
 * whether a shape does; where it does not, smh_partial_rmsnorm is the path. */
int smh_partial_residual_sumsq(const void *partial, int ksplit, int M, int N, const void *h_in, void *h_out, void *sums,
                               smh_stream_t stream);
int smh_q40_norm_in_fits(int M, int K, int nseg, const int *n);
int smh_q40_matmul_partial_tiled_norm(const void *h, long ldh, const void *sums, const void *norm_weight, float eps,
                                      int M, int K, int nseg, const void *const *tiled, const int *n,
                                      void *partial, size_t partial_bytes, smh_stream_t stream);
int smh_partial_reduce(const void *partial, int ksplit, int M, int n_total, int col0, int N, void *c,
                       long ldc, int epilogue, const void *residual, long ldr, smh_stream_t stream);
int smh_partial_rmsnorm(const void *partial, int ksplit, int M, int N, const void *h_in,
                        const void *weight, float eps, void *h_out, void *xn_out, smh_stream_t stream);
int smh_partial_silu_mul(const void *partial, int ksplit, int M, int n_half, void *out, smh_stream_t stream);
int smh_partial_rope_append_kv(const void *partial, int ksplit, int B, int H, int Hkv, int D,
                               void *q, void *k, void *v, const void *cos_tab, const void *sin_tab,
                               const int32_t *pos_dev, void *cache_k, void *cache_ks, void *cache_v,
                               void *cache_vs, int Smax, const int32_t *t_dev, smh_stream_t stream);

/* ---- small fused ops -----------------------------------------------------------------------
 * smh_rmsnorm: RMSNorm.forward (hf_model_q40_kv_shared.py:129-134): fp32 normalise -> fp16 ->
 *   * weight -> fp16.  x,out [rows, dim].
 * smh_silu_mul: F.silu(g) * u in fp16 (hf_model_q40_kv_shared.py:434).
 * smh_argmax: greedy pick, lowest index on ties (hf_model_q40.py:517-519). logits [rows, vocab]
 *   fp16 with row stride ld; out int64 [rows].
 * smh_rope_append_kv: apply_rotary_emb (hf_model_q40_kv_shared.py:173-203) to q[B,H,D] and
 *   k[B,Hkv,D] in place with the fp16 cos/sin row of position *pos_dev (+ b * pos_stride rows? no:
 *   all branches share one position), then quantise the rotated k and v[B,Hkv,D] into row
 *   *t_dev of each branch's Q4_0 suffix cache (hf_model_q40_kv_shared.py:365-371).
 *   cos/sin: fp16 tables [T, D/2].  cache_k/v: bytes [Bmax, Smax, Hkv*D/128, 64],
 *   cache_ks/vs: fp16 [Bmax, Smax, Hkv*D/64].  pos_dev, t_dev: int32 on the device so that a
 *   captured graph can be replayed for successive positions.
 * smh_kv_fork: Attention.fork (hf_model_q40_kv_shared.py:282-297): copy branch `origin`'s rows
 *   to branches curr .. curr+forks-1 in one Q4_0 cache (bytes and scales).
 */
int smh_rmsnorm(const void *x, const void *weight, void *out, int rows, int dim, float eps,
                smh_stream_t stream);
int smh_silu_mul(const void *g, const void *u, void *out, long n, smh_stream_t stream);
int smh_argmax(const void *logits, int rows, int vocab, long ld, int64_t *out, smh_stream_t stream);
/* smh_sample_topk: the sampling step of Transformer.generate (hf_model_q40_kv_shared.py:580-589: logits / temperature,
 * torch.topk, F.softmax, torch.multinomial, gather) for fp16 logits [rows, vocab] in one launch: x = fp16(logit /
 * temperature), the top_k largest x (equal values: lowest index first), p = fp16(softmax over them), one candidate per
 * row drawn by inverse CDF over the candidates in descending order with uniform[row] in [0, 1) - the caller's random
 * numbers take the place of torch.multinomial's generator.  1 <= top_k <= 1024, temperature > 0. */
int smh_sample_topk(const void *logits, int rows, int vocab, long ld, float temperature, int top_k,
                    const float *uniform, int64_t *out, smh_stream_t stream);
/* smh_sample_topk_filter: the sampling step of the flat-cache model's generate (hf_model_q40.py:521-533), whose logits are
 * float32 copies of the fp16 values (:476): x = float(logit) / temperature, everything below the top_k-th largest x masked
 * to -inf (so EVERY value equal to the k-th stays a candidate, not only top_k of them; at most 1024 candidates, lowest
 * indices first, are kept), p = float32 softmax, one candidate per row drawn by inverse CDF with uniform[row] as in
 * smh_sample_topk.  logits: the fp16 values [rows, vocab].  1 <= top_k <= 1024, temperature > 0. */
int smh_sample_topk_filter(const void *logits, int rows, int vocab, long ld, float temperature, int top_k,
                           const float *uniform, int64_t *out, smh_stream_t stream);
/* The expansion step of the tree sampler (mcts.py:115-152) without its per-branch Python loop and host round trips.
 * smh_sample_topk_counts: smh_sample_topk where row r makes counts[r] draws with replacement (torch.multinomial with
 *   num_samples = output_counts[1, r], :128): the draws of row r use uniform[o .. o + counts[r]) and fill out[o ..) with
 *   o = counts[0] + ... + counts[r-1].  counts int32 [rows] on the device; at most 1024 rows.  uniform and out hold
 *   n_draws entries: draws beyond them (counts that add up to more) are not made.
 * smh_tree_fork: the bookkeeping of :127-152 for all *curr_b live branches in one launch: per branch, in order, the
 *   distinct drawn tokens in ascending order with their multiplicities (torch.unique, :131); an alive branch keeps the
 *   smallest on its row and opens one new row per further distinct token while rows are left (:141-150).  A new row
 *   receives the origin's token history (results row), token and multiplicity, and the origin's page ids of the
 *   n_rows suffix rows written so far (what Transformer.fork copies as K/V rows, hf_model_q40_kv_shared.py:282-297;
 *   pages may be NULL).  Then column t of every dead row is zeroed (:160).
 *     draws int64 [n_draws] (the sum of cnt over the live branches; draws past n_draws are ignored); tok, cnt int32 [batch_size] = output_counts[0], [1] (:88-89);
 *     alive uint8 [batch_size] = results_mask; curr_b int32 on the device, updated; results int64 [batch_size, ld];
 *     pages int32 [batch_size, pages_stride]; origin int32 [batch_size]: the branch a row was forked from in this call, else -1.
 *   batch_size <= 1024. */
int smh_sample_topk_counts(const void *logits, int rows, int vocab, long ld, float temperature, int top_k,
                           const float *uniform, const int32_t *counts, int64_t *out, int n_draws, smh_stream_t stream);
/* smh_sample_topk_rowtemp: smh_sample_topk_counts with a temperature per row, row_temps fp32 [rows] on the device (a row
 * whose temperature is not positive draws its largest logit every time, lowest index first among equals: the limit of the
 * distribution) - the tree sampler's temp <= 0 mode, where the logits of branch i are divided by a ramp of its multiplicity
 * (mcts.py:110-114).  There the divisor is a float32 TENSOR, which promotes the fp16 logits: quotients, softmax and
 * probabilities are fp32 here too (no fp16 rounding of x or p); the candidates are the top_k largest logits. */
int smh_sample_topk_rowtemp(const void *logits, int rows, int vocab, long ld, const float *row_temps, int top_k,
                            const float *uniform, const int32_t *counts, int64_t *out, int n_draws, smh_stream_t stream);
int smh_tree_fork(const int64_t *draws, int n_draws, int32_t *tok, int32_t *cnt, const uint8_t *alive, int32_t *curr_b, int batch_size,
                  int64_t *results, long ld, int t, int32_t *pages, long pages_stride, int n_rows, int32_t *origin,
                  smh_stream_t stream);
/* smh_tree_step: one whole step of the search loop after the draws (mcts.py:127-175) in one launch, with the step index read
 * on the device so that the launch can be replayed from a captured HIP graph: smh_tree_fork with column t = *t_dev and
 * n_rows = *t_dev (search step t follows t decode steps; a counter outside the row is cut), then smh_detect_terminal on
 * that column (:162), results_len += alive, alive &= !ended (:163-164, alive is updated in place), next_tokens[r] =
 * results[r, t] (the next forward's input, :102) and summary[0] = branches after the step, summary[1] = rows of the whole
 * batch that have ended (:174's two numbers, the only ones the host reads per step).
 *   state int32 [batch_size] = end_stateMachine; results_len int32 [batch_size]; next_tokens int64 [batch_size]; summary int32 [2]. */
int smh_tree_step(const int64_t *draws, int n_draws, int32_t *tok, int32_t *cnt, uint8_t *alive, int32_t *curr_b, int batch_size,
                  int64_t *results, long ld, const int32_t *t_dev, int32_t *pages, long pages_stride, int32_t *origin,
                  int32_t *state, const int64_t *terminal_seq, int seq_len, int64_t eos, int32_t *results_len,
                  int64_t *next_tokens, int32_t *summary, smh_stream_t stream);
/* smh_detect_terminal: detectTerminal (mcts.py:14-28) for `rows` branches in place: state[b] counts the tokens of
 * terminal_seq (int64 [seq_len], "[/PYTHON]" in the reference, mcts.py:12) produced in a row, any other token sends it
 * back to 0; end[b] = 1 when the sequence is complete or token[b] == eos (2 in the reference), and the state of an ended
 * branch is 0.  token int64 [rows], state int32 [rows] (read and written), end uint8 [rows]. */
int smh_detect_terminal(const int64_t *token, int32_t *state, uint8_t *end, const int64_t *terminal_seq, int seq_len,
                        int64_t eos, int rows, smh_stream_t stream);
int smh_rope_append_kv(void *q, void *k, const void *v, int B, int H, int Hkv, int D,
                       const void *cos_tab, const void *sin_tab, const int32_t *pos_dev,
                       void *cache_k, void *cache_ks, void *cache_v, void *cache_vs,
                       int Smax, const int32_t *t_dev, smh_stream_t stream);
int smh_rope(void *q, void *k, int S, int H, int Hkv, int D, const void *cos_tab,
             const void *sin_tab, int pos0, smh_stream_t stream);
int smh_kv_fork(void *cache, void *cache_s, int Bmax, long row_bytes, long row_scales,
                int origin, int curr, int forks, smh_stream_t stream);
/* smh_set_step: state[0] = pos, state[1] = t (int32 on the device), the `start_pos` of Transformer.forward
 * (hf_model_q40_kv_shared.py:492) and the suffix row start_pos - prompt length (:333-336) that the decode kernels read
 * through pos_dev / t_dev.  The values travel as kernel arguments: no host buffer, no copy, nothing the host waits for. */
int smh_set_step(int32_t *state, int pos, int t, smh_stream_t stream);

/* ---- fp16 vocabulary projection and embedding -------------------------------------------------------
 * smh_f16_linear: out[M, N] = x[M, K] . w[N, K]^T, fp16 operands, fp32 accumulation, one rounding to fp16: the
 *   `self.output(h)` of Transformer.forward (hf_model_q40_kv_shared.py:509; nn.Linear without bias, weight [vocab, dim]
 *   as the checkpoint holds it, :484).  x rows ldx apart, out rows ldo apart; K % 64 == 0, ldx % 8 == 0, x and w 16-byte
 *   aligned.  N need not be a multiple of anything (vocab 32016).
 * smh_embedding: out[m, :] = table[tokens[m], :], the `self.tok_embeddings(tokens)` of Transformer.forward (:495; table
 *   [vocab, dim] fp16, :477).  tokens int64 [M] on the device; dim % 8 == 0. */
int smh_f16_linear(const void *x, int M, int K, long ldx, const void *w, int N, void *out, long ldo, smh_stream_t stream);
int smh_embedding(const int64_t *tokens, int M, const void *table, int vocab, int dim, void *out, smh_stream_t stream);

/* ---- attention -----------------------------------------------------------------------------
 * smh_shared_prefix_attn: the decode attention of Attention.forward
 * (hf_model_q40_kv_shared.py:375-405) without materialising or copying the prefix per branch:
 * out[b,h,:] = softmax(q[b,h,:] . K_b^T / sqrt(D)) . V_b  with  K_b = [prefix (P rows, shared) ||
 * suffix of branch b (lens[b] rows) || cur_k[b] (one exact fp16 row, optional)].
 *   q, out      fp16 [B, H, D], D == 128
 *   prefix_k/v  fp16 [P, Hkv, D]
 *   suffix      SMH_KV_FP16: suffix_k/v fp16 [B, Smax, Hkv, D]
 *               SMH_KV_Q40 : suffix_k/v bytes [B, Smax, Hkv*D/128, 64], suffix_ks/vs fp16 [B, Smax, Hkv*D/64]
 *   lens        int32 [B] on the device (rows of the suffix that are valid); with len_offset
 *               added to each (the model passes the step counter t for every branch)
 *   cur_k/v     fp16 [B, Hkv, D] or NULL
 *   workspace   smh_attn_workspace_bytes(B, H, P) bytes of scratch (no initialisation needed)
 * smh_prefill_attn: causal attention over the prompt (hf_model_q40_kv_shared.py:499-504,405),
 *   q [S,H,D], k,v [S,Hkv,D] -> out [S,H,D].
 */
size_t smh_attn_workspace_bytes(int B, int H, int P);
int smh_shared_prefix_attn(const void *q, void *out, int B, int H, int Hkv, int D,
                           const void *prefix_k, const void *prefix_v, int P,
                           int suffix_format, const void *suffix_k, const void *suffix_v,
                           const void *suffix_ks, const void *suffix_vs, int Smax,
                           const int32_t *lens, int lens_stride, const void *cur_k, const void *cur_v,
                           void *workspace, size_t workspace_bytes, smh_stream_t stream);
int smh_prefill_attn(const void *q, const void *k, const void *v, void *out, int S, int H, int Hkv,
                     int D, smh_stream_t stream);

/* ---- paged / tree attention --------------------------------------------------------------------------------------
 * smh_paged_prefix_attn: smh_shared_prefix_attn whose per-branch rows are looked up in a page table inside the
 * kernel, one token per page: the reference's tree attention page_flash_attn (triton_kernels.py:649-789, pager[B, L] ->
 * page pool) and the intent of chunk_attn (:1150-1231: a shared first chunk, then the branch's own pages).  Branches
 * forked from a common ancestor share the ancestor's pages, so Attention.fork (hf_model_q40_kv_shared.py:282-297)
 * becomes a copy of page ids (smh_page_fork) instead of a copy of K/V rows.
 *   out[b,h,:] = softmax(q[b,h,:] . K_b^T / sqrt(D)) . V_b,  K_b = [prefix rows 0..P-1 (shared) || pool rows
 *                pages[b, 0 .. lens[b]-1] || cur_k[b] (optional)]
 *   prefix_k/v   fp16, element strides prefix_row_stride between rows and prefix_head_stride between kv heads
 *                (0, 0 = token-major [P, Hkv, D]; a head-major pool [Hkv, rows, D] is (D, rows * D))
 *   pool         SMH_KV_FP16: pool_k/v fp16 with pool_row_stride / pool_head_stride as above;
 *                SMH_KV_Q40: the model's cache rows, bytes [rows, Hkv, 64] + scales fp16 [rows, Hkv, 2] (strides 0)
 *   pages        page ids of page_bytes = 2, 4 or 8 bytes each (int16 as in the reference, int32, int64): row b starts at
 *                element b * pages_stride and holds pages_cols ids (a column slice of a wider table has pages_cols <
 *                pages_stride); lens[b] is cut to pages_cols, so no id past a row's end is read;
 *                the pool has pool_rows rows: an id outside 0 .. pool_rows-1 is read as the nearest valid row (a wrong
 *                result for that branch, never an access outside the pool)
 *   lens         int32 [B] (lens_stride 1) or one shared int32 (lens_stride 0): pages of the branch that are valid
 *   single_launch, workspace: as smh_shared_prefix_attn_one (counters zeroed once) when != 0, else as smh_shared_prefix_attn
 * smh_page_fork: table[curr + i, 0..n-1] = table[origin, 0..n-1] for i < forks; table int32 [rows, stride]. */
int smh_paged_prefix_attn(const void *q, void *out, int B, int H, int Hkv, int D,
                          const void *prefix_k, const void *prefix_v, int P, long prefix_row_stride, long prefix_head_stride,
                          int pool_format, const void *pool_k, const void *pool_v, const void *pool_ks, const void *pool_vs,
                          long pool_row_stride, long pool_head_stride, long pool_rows,
                          const void *pages, int page_bytes, long pages_stride, int pages_cols, const int32_t *lens, int lens_stride,
                          const void *cur_k, const void *cur_v, int single_launch,
                          void *workspace, size_t workspace_bytes, smh_stream_t stream);
int smh_page_fork(int32_t *table, int rows, long stride, int origin, int curr, int forks, int n, smh_stream_t stream);

/* smh_shared_prefix_attn_static: smh_shared_prefix_attn (same arguments without the workspace, same kernels, bit-identical
 * results) for callers that cannot allocate device memory or pass a workspace: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  The prefix partials live in
 * a static device array of smh_attn_static_scratch_bytes() = 16 MiB that every GPU the library runs on holds until the
 * process ends; shapes that need more (prefix slices x B x H x 520 bytes) are rejected with an error.  The call allocates
 * and frees nothing; the first call on a device looks the array's address up (make that call outside a graph capture).
 * All calls on one GPU share the array: calls that overlap in time on one GPU race - keep them on one stream. */
size_t smh_attn_static_scratch_bytes(void);
int smh_shared_prefix_attn_static(const void *q, void *out, int B, int H, int Hkv, int D,
                                  const void *prefix_k, const void *prefix_v, int P,
                                  int suffix_format, const void *suffix_k, const void *suffix_v,
                                  const void *suffix_ks, const void *suffix_vs, int Smax,
                                  const int32_t *lens, int lens_stride, const void *cur_k, const void *cur_v,
                                  smh_stream_t stream);

/* smh_shared_prefix_attn_one: smh_shared_prefix_attn (same arguments, same attention) in ONE launch instead of
 * two: prefix slices and the branches' suffix passes run side by side and the workgroup that completes a
 * tile of 16 queries merges its partials in a fixed order (deterministic; equal to the two-launch result up
 * to fp32 summation order).  B * (H / Hkv) <= 128.  workspace: smh_attn_qkv_workspace_bytes(B, H, P) bytes whose
 * first 4096 bytes (arrival counters) are zero before the first call; the calls leave them zero.  Calls that
 * overlap in time need separate workspaces. */
int smh_shared_prefix_attn_one(const void *q, void *out, int B, int H, int Hkv, int D,
                               const void *prefix_k, const void *prefix_v, int P,
                               int suffix_format, const void *suffix_k, const void *suffix_v,
                               const void *suffix_ks, const void *suffix_vs, int Smax,
                               const int32_t *lens, int lens_stride, const void *cur_k, const void *cur_v,
                               void *workspace, size_t workspace_bytes, smh_stream_t stream);

/* smh_shared_prefix_attn_qkv: smh_partial_rope_append_kv + smh_shared_prefix_attn without the RoPE launch, for up
 * to 16 branches: the attention kernels take q and the new token's k, v straight from the slabs of the
 * wq|wk|wv product (smh_q40_matmul_partial with the three weights as segments; B <= 16, so fp32 slabs),
 * apply apply_rotary_emb (hf_model_q40_kv_shared.py:173-203) at position *pos_dev, append Q4_0(k), Q4_0(v)
 * to row *t_dev of every branch's suffix cache (:365-371) and attend over prefix (P rows) || suffix rows
 * 0 .. *t_dev - 1 of the branch (the Q4_0 cache) || the new token (exact fp16).  q, k, v are not
 * materialised.  B * (H / Hkv) <= 128.
 *   single_launch == 0: two launches (prefix slices, then suffix + merge), same rounding points and summation
 *                       order as the three-launch sequence: results are bit-identical to it;
 *                       workspace as for smh_shared_prefix_attn.
 *   single_launch != 0: ONE launch: prefix slices and the branches' suffixes run side by side, the workgroup
 *                       that completes the count of a tile of 16 queries merges its partials in a fixed order
 *                       (the faster form up to about 16 queries per kv head, B * H / Hkv; above, the one workgroup
 *                       that merges a kv head's tiles takes longer than a second launch).
 *                       workspace: smh_attn_qkv_workspace_bytes(B, H, P) bytes whose first 4096 bytes (the
 *                       counters) are zero before the first call; the calls leave them zero.  Calls that
 *                       overlap in time need separate workspaces.
 *   pages               NULL, or a page table int32 [B, pages_stride] (pages_stride >= Smax): suffix row j of branch b is
 *                       read from cache row pages[b * pages_stride + j] (rows counted over all branches, i.e. branch b's own
 *                       row j is b * Smax + j) - branches forked from a common ancestor share its rows instead of holding
 *                       copies (see smh_paged_prefix_attn).  The new token's row is still appended at b * Smax + *t_dev. */
size_t smh_attn_qkv_workspace_bytes(int B, int H, int P);
int smh_shared_prefix_attn_qkv(const void *qkv_partial, int ksplit, void *out, int B, int H, int Hkv, int D,
                               const void *cos_tab, const void *sin_tab, const int32_t *pos_dev,
                               const void *prefix_k, const void *prefix_v, int P,
                               void *cache_k, void *cache_ks, void *cache_v, void *cache_vs, int Smax,
                               const int32_t *t_dev, const int32_t *pages, int pages_stride, int single_launch,
                               void *workspace, size_t workspace_bytes, smh_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* SMH_H */
