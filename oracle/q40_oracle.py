"""CPU oracle for the Q4_0 CodeLlama hot path.  TEST INFRASTRUCTURE ONLY.

This module restates, in plain torch-on-CPU / numpy, the arithmetic of the reference's Q4_0
inference path so that the HIP kernels can be checked against it.  It is never imported by the
product package: only `tests/`, `__graft_entry__.smoke()` and the `cpu_baseline` leg of
`bench.py` may use it, and only as the checker or as the timed CPU baseline.

Every function cites the reference lines it follows (paths relative to the reference checkout).

Parity pins (what fixes each function independently of this file's own formulas; the checks
live in tests/test_oracle_*.py):
  quantize_q40 / dequantize_q40  exhaustive 16 nibbles x 65536 fp16 scale patterns against an
                                 integer-only C restatement (oracle/q40_ref.c) and numpy float16;
                                 quantiser invariants (code range, |err| <= scale/2, idempotence),
                                 brute force on tiny groups with exact rationals.
  quantize_gq40 / dequantize_gq40  (the block-of-32 flavour of the benchmark's first configuration; no counterpart in the
                                 reference's code) every (nibble, fp16 scale) pair against integer arithmetic on the
                                 bit patterns; |error| <= scale / 2 except at +absmax (cut from 16 to 15: one scale);
                                 re-quantising a dequantised tensor reproduces the codes.
  weight layout                  closed-form byte map  byte(k, (n//128)*64 + n%64), high nibble
                                 iff n%128 < 64, scale s[k, n//64]  checked element by element.
  matmul_q40                     float64 dense matmul of the dequantised matrix; one-hot inputs
                                 return single dequantised rows bit-exactly.
  rmsnorm / rope / silu          textbook closed forms evaluated in float64 (position 0 is the
                                 identity, pairwise norm preservation, table = cos/sin(t*theta^-2i/d)).
  shared_prefix_attention        torch.nn.functional.scaled_dot_product_attention on the
                                 concatenated K/V (library routine), uniform scores -> mean of V,
                                 one dominant key -> that V row, invariance to the split point.
  OracleTransformer              composition only; cross-checked by (i) dense-weight F.linear model,
                                 (ii) prefill-vs-incremental equality with KV quantisation off,
                                 (iii) identical branches give identical tokens.
  topk_probs / sample_topk       candidate values against torch.topk, probabilities against F.softmax of those values,
                                 k = 1 is the argmax, k = vocab with a huge temperature is uniform; the draw against a
                                 brute-force scan in float64 and, over many uniform numbers, its frequencies against p.
  sample_topk_counts / tree_fork the draws against sample_topk row by row; the bookkeeping against hand-computed known answers
                                 (every row of a small tree written out), conservation of the multiplicities while rows are
                                 left, truncation when they run out, dead branches untouched, histories of forked rows.
  detect_terminal                a scalar walk over token streams written as plain if / else (tests), known answers:
                                 the sequence fed in order ends at its last token, end-of-sequence ends at once, a
                                 wrong token resets, a repeated first token does NOT restart the match (the reference's
                                 behaviour), every (state, token-class) pair enumerated.
No function here is "parity unpinned".
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import numpy as np
import torch
import torch.nn.functional as F

GROUP_SIZE = 64
DTYPE = torch.float16


# --------------------------------------------------------------------------------------------
# Q4_0 codec  (fp16_to_int4.py:52-96; same maths at triton_kernels.py:12-56,
#              hf_model_q40_kv_shared.py:74-118, hf_model_q40.py:71-115)
# --------------------------------------------------------------------------------------------
def quantize_q40(w: torch.Tensor, group_size: int = GROUP_SIZE) -> Tuple[torch.Tensor, torch.Tensor]:
    """Symmetric 4-bit quantisation, codes in [-7, 7], fp16 scale = absmax/7 per 64 values.

    Two consecutive groups share one 64-byte row: group 2p in the high nibbles, group 2p+1 in the
    low nibbles (fp16_to_int4.py:73-79).  Returns (int8 [numel/128, 64], fp16 [numel/64, 1]).
    """
    assert w.numel() % (2 * group_size) == 0
    w = w.reshape(-1, group_size)
    wmax = torch.abs(w).max(dim=1).values
    scale = (wmax / 7.0).type(DTYPE)[:, None]          # fp16_to_int4.py:63-65
    quant = w / scale                                  # fp16 / fp16 -> fp16 (bf16/fp32 promote)
    int8val = torch.round(quant).to(torch.int8)        # half-to-even; 0/0 -> NaN -> 0
    pair = int8val.reshape(-1, 2, group_size)
    msb, lsb = pair[:, 0, :], pair[:, 1, :]
    packed = (msb << 4) | (lsb & 0x0F)                 # fp16_to_int4.py:78
    return packed.reshape(-1, group_size).contiguous(), scale


def dequantize_q40(w: torch.Tensor, scale: torch.Tensor, group_size: int, shape, ptdtype=DTYPE) -> torch.Tensor:
    """Sign-extending nibble unpack followed by ONE fp16 multiply (fp16_to_int4.py:90-96).

    `w >> 4` is arithmetic on int8; `(w << 4) >> 4` wraps in int8 then shifts arithmetically, so
    nibble 0x8 decodes to -8.  hstack puts the high-nibble group first.
    """
    msb = w >> 4
    lsb = (w << 4) >> 4
    q = torch.hstack((msb, lsb)).view(-1, group_size)
    return (q * scale.view(-1, 1)).type(ptdtype).reshape(shape)


# The OTHER Q4_0 flavour: the one the benchmark's first configuration spells out in words (32-weight blocks along the input
# dimension, one fp16 scale = absmax / 8 per block, nibbles q in [0, 15] packed two per byte, value = (q - 8) * scale).
# The reference's code has no such format (its Q4_0 is the 64-group, absmax / 7, signed-nibble layout above); this is a
# restatement of that text, with the arithmetic conventions of the reference's own quantiser where the text is silent:
# the scale is fp16(absmax / 8.0), the quotient w / scale is an fp16 division, codes round half to even, 0 / 0 gives q = 8,
# and element j of a block shares byte j with element j + 16 (low nibble, high nibble) as the widespread block format does.
GQ_BLOCK = 32


def quantize_gq40(w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """w fp16 [..., K] with K % 32 == 0 -> (packed uint8 [numel/32, 16], scale fp16 [numel/32])."""
    assert w.dtype == DTYPE and w.shape[-1] % GQ_BLOCK == 0
    blocks = w.reshape(-1, GQ_BLOCK)
    scale = (blocks.abs().max(dim=1).values / 8.0).type(DTYPE)
    quot = blocks / scale[:, None]                                   # fp16 / fp16
    # (a scale that underflows to 0 under a non-zero block gives +-inf: cut like any quotient outside the code range)
    q = torch.nan_to_num(torch.round(quot).float(), nan=0.0, posinf=8.0, neginf=-8.0).clamp(-8.0, 8.0).to(torch.int32) + 8
    q = q.clamp(0, 15)                                               # +absmax maps to 16: cut to 15
    packed = (q[:, :16] | (q[:, 16:] << 4)).to(torch.uint8)
    return packed.contiguous(), scale


def dequantize_gq40(packed: torch.Tensor, scale: torch.Tensor, shape) -> torch.Tensor:
    """value = (q - 8) * scale, ONE fp16 multiply per weight."""
    p32 = packed.to(torch.int32)
    q = torch.cat((p32 & 15, p32 >> 4), dim=1) - 8                   # [blocks, 32]
    return (q.to(torch.int8) * scale.view(-1, 1)).type(DTYPE).reshape(shape)


def linear_gq40(x: torch.Tensor, packed: torch.Tensor, scale: torch.Tensor, shape) -> torch.Tensor:
    """y = x . W^T with W [N, K] held in the block format: dequantise to fp16, accumulate in fp32, round once."""
    return (x.float() @ dequantize_gq40(packed, scale, shape).float().t()).to(DTYPE)


def unpack_codes(w: torch.Tensor) -> torch.Tensor:
    """int8 codes in group order ([numel/64, 64]) without scaling (helper for tests)."""
    msb = w >> 4
    lsb = (w << 4) >> 4
    return torch.hstack((msb, lsb)).view(-1, GROUP_SIZE)


def quantize_weight(v: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Size]:
    """Checkpoint conversion of one linear weight v[N_out, K_in]: quantise the TRANSPOSE so a
    scale group is 64 consecutive outputs n at fixed k (fp16_to_int4.py:173-176)."""
    w, s = quantize_q40(v.t(), GROUP_SIZE)
    return w, s, v.shape


def weight_byte_index(k: int, n: int, N: int) -> Tuple[int, bool, int]:
    """Closed form of the layout produced by quantize_weight: (flat byte index into w.view(-1),
    is_high_nibble, flat scale index into s.view(-1)) for logical element W^T[k, n].
    Kernel views are w.view(K, N//2) and s.view(K, N//64) (triton_kernels.py:481-482)."""
    byte = k * (N // 2) + (n // 128) * 64 + (n % 64)
    return byte, (n % 128) < 64, k * (N // 64) + n // 64


# --------------------------------------------------------------------------------------------
# Q4_0 linear
# --------------------------------------------------------------------------------------------
def matmul_q40(a: torch.Tensor, b_w: torch.Tensor, b_s: torch.Tensor, b_shape) -> torch.Tensor:
    """C[M,N] = A[M,K] . deq(B)[K,N]: operands dequantised to fp16, products accumulated in
    fp32, one rounding to fp16 (triton_kernels.py:444-449,464,471-500)."""
    K, N = b_shape
    assert a.shape[1] == K
    deq = dequantize_q40(b_w, b_s, GROUP_SIZE, (K, N), DTYPE)
    return (a.float() @ deq.float()).to(DTYPE)


def linear_q40_cpu_path(x: torch.Tensor, w: torch.Tensor, s: torch.Tensor, shape) -> torch.Tensor:
    """The reference's torch-only linear: dequantise the whole weight, then F.linear
    (hf_model_q40.py:222-226).  `shape` is what the checkpoint stores: (N_out, K_in); with the
    transposed checkpoint flavour the dequantised matrix is [K, N], hence the transpose.
    Used as the timed CPU baseline; fp32 compute because CPU fp16 GEMM is not a fast path."""
    N, K = shape
    deq = dequantize_q40(w, s, GROUP_SIZE, (K, N), DTYPE)
    return F.linear(x.float(), deq.t().float()).to(DTYPE)


# --------------------------------------------------------------------------------------------
# Small ops (hf_model_q40_kv_shared.py:123-203, 431-436)
# --------------------------------------------------------------------------------------------
def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """fp32 normalise -> cast to x.dtype -> * weight -> cast (hf_model_q40_kv_shared.py:129-134)."""
    xf = x.float()
    out = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).type_as(x)
    return (out * weight).type_as(x)


def precompute_freqs_cis(dim: int, end: int, theta: float) -> torch.Tensor:
    """complex64 [end, dim/2] rotation table (hf_model_q40_kv_shared.py:137-142)."""
    freqs = 1.0 / (theta ** (torch.arange(0, dim, 2)[: (dim // 2)].float() / dim))
    t = torch.arange(end, dtype=torch.float32)
    freqs = torch.outer(t, freqs)
    return torch.polar(torch.ones_like(freqs), freqs)


def rope_tables_fp16(freqs_cis: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """cos/sin rounded to fp16 and duplicated to the full head dim
    (hf_model_q40_kv_shared.py:193-196)."""
    cos = freqs_cis.real.to(DTYPE)
    sin = freqs_cis.imag.to(DTYPE)
    return torch.cat((cos, cos), dim=1), torch.cat((sin, sin), dim=1)


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    x1 = x[..., : x.shape[-1] // 2]
    x2 = x[..., x.shape[-1] // 2:]
    return torch.cat((-x2, x1), dim=-1)


def apply_rotary_emb(q: torch.Tensor, k: torch.Tensor, freqs_cis: torch.Tensor):
    """q,k: [B, S, H, D] fp16; three fp16 roundings per element: q*cos, rot(q)*sin, sum
    (hf_model_q40_kv_shared.py:173-203)."""
    cos, sin = rope_tables_fp16(freqs_cis)             # [S, D]
    cos = cos[None, :, None, :]
    sin = sin[None, :, None, :]
    q_embed = (q * cos) + (rotate_half(q) * sin)
    k_embed = (k * cos) + (rotate_half(k) * sin)
    return q_embed, k_embed


def ramp_temperature(temp: float, batch_size: int, counts: torch.Tensor) -> torch.Tensor:
    """The per-branch temperature of the tree sampler's temp <= 0 mode (mcts.py:113, the lambda f applied to
    output_counts[1, :curr]): a line from 0.1 at multiplicity 1 to |temp| at multiplicity batch_size; counts int32 ->
    float32, as torch promotes int32 * Python float."""
    return (abs(temp) - 0.1) / (batch_size - 1) * (counts - 1) + 0.1


def topk_probs(logits: torch.Tensor, temperature, top_k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """The candidates of the reference's sampling step (hf_model_q40_kv_shared.py:580-586): `logits / temperature` on
    the fp16 tensor, `torch.topk`, `F.softmax` (fp16 in, fp16 out).  Returns (p [rows, k] fp16, idx [rows, k]) in
    descending order of value; equal values are ordered by index (torch.topk leaves that order open).
    temperature may be a float32 tensor [rows] (mcts.py:114, `(logits.t() / f(..)).t()`): torch then promotes the
    quotient, and with it the softmax, to float32."""
    if isinstance(temperature, torch.Tensor):
        x = (logits.t() / temperature).t()                     # fp16 tensor / fp32 tensor: fp32 result
        k = min(top_k, x.shape[-1])
        order = torch.argsort(x, dim=-1, descending=True, stable=True)[:, :k]
        return F.softmax(torch.gather(x, 1, order), dim=-1), order
    x = logits / temperature                                   # fp16 tensor / python float: fp16 result
    k = min(top_k, x.shape[-1])
    order = torch.argsort(x.float(), dim=-1, descending=True, stable=True)[:, :k]
    v = torch.gather(x, 1, order)
    return F.softmax(v, dim=-1), order


def sample_topk(logits: torch.Tensor, temperature: float, top_k: int, u: torch.Tensor) -> torch.Tensor:
    """One draw per row from topk_probs by inverse CDF with the given uniform numbers u [rows] in [0, 1): the first
    candidate (descending order) whose cumulative probability exceeds u * total.  Stands in for `torch.multinomial`
    (:588), whose generator cannot be reproduced: same distribution, the caller's randomness."""
    p, order = topk_probs(logits, temperature, top_k)
    cdf = p.float().cumsum(-1)
    target = u.float().unsqueeze(1) * cdf[:, -1:]
    hit = cdf > target
    j = torch.where(hit.any(-1), hit.float().argmax(-1), torch.full((p.shape[0],), p.shape[1] - 1))
    return order.gather(1, j.unsqueeze(1))[:, 0]


def topk_filter_probs(logits: torch.Tensor, temperature: float, top_k: int) -> torch.Tensor:
    """The probabilities of the flat-cache model's sampling step (hf_model_q40.py:521-529): float32 logits (that model
    returns `output.float()`, :476) divided by the temperature, every value below the top_k-th largest set to -inf - values
    equal to it all stay, so more than top_k may survive - and a float32 softmax over the vocabulary.  [rows, vocab]."""
    x = logits.float() / temperature
    v, _ = torch.topk(x, min(top_k, x.size(-1)))
    x = x.masked_fill(x < v[:, [-1]], -float("Inf"))
    return F.softmax(x, dim=-1)


def sample_topk_filter(logits: torch.Tensor, temperature: float, top_k: int, u: torch.Tensor) -> torch.Tensor:
    """One draw per row from topk_filter_probs by inverse CDF over the surviving tokens in descending order of value (equal
    values by index), with the caller's uniform numbers - the stand-in for `torch.multinomial` (:530) that sample_topk
    uses."""
    p = topk_filter_probs(logits, temperature, top_k)
    order = torch.argsort(logits.float(), dim=-1, descending=True, stable=True)
    ps = torch.gather(p, 1, order)
    cdf = ps.cumsum(-1)
    n_alive = (ps > 0).sum(-1)
    total = cdf.gather(1, (n_alive - 1).unsqueeze(1))
    hit = cdf > u.float().unsqueeze(1) * total
    j = torch.where(hit.any(-1), hit.float().argmax(-1), n_alive - 1)
    return order.gather(1, j.unsqueeze(1))[:, 0]


def sample_topk_counts(logits: torch.Tensor, temperature, top_k: int, counts, u: torch.Tensor) -> torch.Tensor:
    """counts[r] draws per row (mcts.py:128: torch.multinomial(probs[r], num_samples=output_counts[1, r], replacement=True)
    followed by the gather of :129), each an inverse-CDF draw as in sample_topk; row r uses u[sum(counts[:r]) ...]."""
    out = []
    off = 0
    for r in range(logits.shape[0]):
        n = int(counts[r])
        if n:
            tr = temperature[r:r + 1].expand(n) if isinstance(temperature, torch.Tensor) else temperature
            out.append(sample_topk(logits[r:r + 1].expand(n, -1), tr, top_k, u[off:off + n]))
        off += n
    return torch.cat(out) if out else torch.zeros(0, dtype=torch.int64)


def tree_fork(draws: torch.Tensor, output_counts: torch.Tensor, alive: torch.Tensor, curr_batch: int, batch_size: int,
              results: torch.Tensor, t: int, pages: Optional[torch.Tensor] = None, n_rows: int = 0):
    """The per-branch loop of the tree sampler's expansion step (mcts.py:127-152) and the masking of :160, on host tensors,
    in place.  draws: the tokens the live branches sampled, branch after branch (output_counts[1, i] each).  Returns
    (new curr_batch, origin list: the branch each row was forked from in this call, else -1)."""
    origin = [-1] * batch_size
    off = 0
    segs = []
    for i in range(curr_batch):
        n = int(output_counts[1, i])
        segs.append(draws[off:off + n])
        off += n
    for i in range(curr_batch):
        next_token = segs[i]
        if next_token.numel() == 0:
            continue
        unique_idx, counts = torch.unique(next_token, return_counts=True, dim=0)      # ascending (:131)
        if alive[i]:                                                                 # :135-138
            output_counts[0, i] = unique_idx[0]
            output_counts[1, i] = counts[0]
            results[i, t] = unique_idx[0]
        forks = min(len(counts) - 1, batch_size - curr_batch)                        # :141-142
        if forks > 0 and curr_batch < batch_size and alive[i]:                       # :143
            for j in range(forks):                                                   # model.fork(i, curr_batch, forks) + :146-150
                r = curr_batch + j
                origin[r] = i
                if pages is not None:
                    pages[r, :n_rows] = pages[i, :n_rows]
                results[r] = results[i]
                output_counts[0, r] = unique_idx[1 + j]
                output_counts[1, r] = counts[1 + j]
                results[r, t] = unique_idx[1 + j]
            curr_batch += forks
    results[:, t] *= alive.to(results.dtype)                                         # :160
    return curr_batch, origin


def detect_terminal(token: torch.Tensor, state: torch.Tensor, terminal_seq: torch.Tensor, eos: int = 2):
    """detectTerminal (mcts.py:14-28): mask = terminal_seq[state] == token; state = (state + mask) * mask;
    end = state == len(terminal_seq) or token == eos; an ended branch restarts at state 0.
    token int64 [B], state int32 [B] -> (end bool [B], state int32 [B])."""
    mask = (terminal_seq.gather(0, state.to(torch.int64)) == token).to(torch.int32)
    state = (state + mask) * mask
    end = (state == terminal_seq.numel()) | (token == eos)
    return end, (~end).to(torch.int32) * state


def silu_mul(g: torch.Tensor, u: torch.Tensor) -> torch.Tensor:
    """F.silu(w1 x) * w3 x in fp16: silu rounds to fp16, the product rounds again
    (hf_model_q40_kv_shared.py:434)."""
    return F.silu(g.float()).to(g.dtype) * u


# --------------------------------------------------------------------------------------------
# Attention
# --------------------------------------------------------------------------------------------
def shared_prefix_attention(q: torch.Tensor, prefix_k: torch.Tensor, prefix_v: torch.Tensor,
                            suffix_k: Optional[torch.Tensor], suffix_v: Optional[torch.Tensor],
                            lens: Optional[List[int]], acc_dtype=torch.float32, p_half_prefix: bool = False) -> torch.Tensor:
    """One query per branch over [shared prefix || that branch's own suffix].

    q [B,H,D]; prefix_k/v [P,Hkv,D]; suffix_k/v [B,S,Hkv,D] with lens[b] valid rows.
    softmax(q.K^T/sqrt(D)).V with fp32 scores/softmax/accumulation, fp16 result: what
    F.scaled_dot_product_attention computes at hf_model_q40_kv_shared.py:375-405 (there the prefix
    is expanded per branch and all lens are equal).
    The two keyword arguments are instruments for noise studies, not part of the reference's arithmetic: `acc_dtype`
    float64 evaluates the same formula in double precision; `p_half_prefix` rounds the un-normalised probabilities of the
    PREFIX keys to fp16 before they multiply V (what a matrix-core P.V product with fp16 operands does), the
    denominator keeping the unrounded values."""
    B, H, D = q.shape
    Hkv = prefix_k.shape[1]
    n_rep = H // Hkv
    P = prefix_k.shape[0]
    out = torch.empty((B, H, D), dtype=q.dtype)
    for b in range(B):
        k = prefix_k
        v = prefix_v
        if suffix_k is not None and lens is not None and lens[b] > 0:
            k = torch.cat((k, suffix_k[b, : lens[b]]), dim=0)
            v = torch.cat((v, suffix_v[b, : lens[b]]), dim=0)
        kf = k.to(acc_dtype).repeat_interleave(n_rep, dim=1)       # [L, H, D]
        vf = v.to(acc_dtype).repeat_interleave(n_rep, dim=1)
        scores = torch.einsum("hd,lhd->hl", q[b].to(acc_dtype), kf) / math.sqrt(D)
        if not p_half_prefix:
            p = torch.softmax(scores, dim=-1)
        else:
            e = torch.exp(scores - scores.max(dim=-1, keepdim=True).values)
            den = e.sum(dim=-1, keepdim=True)
            e = torch.cat((e[:, :P].to(DTYPE).to(acc_dtype), e[:, P:]), dim=1)
            p = e / den
        out[b] = torch.einsum("hl,lhd->hd", p, vf).to(q.dtype)
    return out


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, acc_dtype=torch.float32, p_half: bool = False) -> torch.Tensor:
    """Prefill attention: q,k,v [S,H(kv),D]; additive -inf above the diagonal
    (hf_model_q40_kv_shared.py:499-504, 405).  acc_dtype / p_half: as in shared_prefix_attention (noise studies)."""
    S, H, D = q.shape
    n_rep = H // k.shape[1]
    kf = k.to(acc_dtype).repeat_interleave(n_rep, dim=1)
    vf = v.to(acc_dtype).repeat_interleave(n_rep, dim=1)
    scores = torch.einsum("shd,lhd->hsl", q.to(acc_dtype), kf) / math.sqrt(D)
    mask = torch.full((S, S), float("-inf"), dtype=acc_dtype).triu(diagonal=1)
    scores = scores + mask
    if not p_half:
        p = torch.softmax(scores, dim=-1)
    else:
        e = torch.exp(scores - scores.max(dim=-1, keepdim=True).values)
        p = e.to(DTYPE).to(acc_dtype) / e.sum(dim=-1, keepdim=True)
    return torch.einsum("hsl,lhd->shd", p, vf).to(q.dtype)


# --------------------------------------------------------------------------------------------
# Whole model (hf_model_q40_kv_shared.py:252-510)
# --------------------------------------------------------------------------------------------
@dataclass
class OracleArgs:
    dim: int = 4096
    n_layers: int = 32
    n_heads: int = 32
    n_kv_heads: Optional[int] = None
    vocab_size: int = 32016
    multiple_of: int = 256
    ffn_dim_multiplier: Optional[float] = None
    norm_eps: float = 1e-5
    rope_theta: float = 1000000.0
    max_batch_size: int = 80
    max_seq_len: int = 256
    max_prompt_seq_len: int = 256


def ffn_hidden_dim(dim: int, multiple_of: int, ffn_dim_multiplier: Optional[float]) -> int:
    """hf_model_q40_kv_shared.py:421-425 with hidden_dim = 4*dim (:448)."""
    hidden = int(2 * (4 * dim) / 3)
    if ffn_dim_multiplier is not None:
        hidden = int(ffn_dim_multiplier * hidden)
    return multiple_of * ((hidden + multiple_of - 1) // multiple_of)


class OracleTransformer:
    """Functional restatement of Transformer.forward with the shared fp16 prompt KV cache and the
    per-branch Q4_0 suffix KV cache.  `sd` uses the checkpoint's key names:
    tok_embeddings.weight, norm.weight, output.weight, layers.{i}.attention_norm.weight,
    layers.{i}.ffn_norm.weight and layers.{i}.{attention.wq|wk|wv|wo, feed_forward.w1|w2|w3}.{w,s,shape}.

    With `dense=True` the quantised linears are replaced once by their dequantised fp32 matrices
    (identical values, much faster per step); `quantize_kv=False` keeps the suffix KV in fp16.
    """

    LINEARS = ("attention.wq", "attention.wk", "attention.wv", "attention.wo",
               "feed_forward.w1", "feed_forward.w2", "feed_forward.w3")

    def __init__(self, args: OracleArgs, sd: Dict[str, torch.Tensor], dense: bool = True,
                 quantize_kv: bool = True, per_branch_kv: bool = False, acc_dtype=torch.float32,
                 scale_on_x_max_rows: int = 0, p_half_prefix: bool = False, slab_half_ksplit=None, share_dense=None):
        # The last five arguments are instruments for noise studies (how far may two faithful implementations of the
        # same cast points drift apart on a deep random model), not the reference's arithmetic; the defaults are the oracle.
        #   acc_dtype float64        every matrix product and the attention accumulate in double precision
        #   scale_on_x_max_rows = R  linears of at most R rows round fp16(x * scale) and multiply by the integer code,
        #                            instead of x by fp16(code * scale): same values before rounding, the rounding on the other operand
        #   p_half_prefix            see shared_prefix_attention (prefill: all keys)
        #   slab_half_ksplit(key, K, N) -> number of K-slices whose partial sums are rounded to fp16 before they are added
        #   share_dense              another oracle whose dequantised matrices are reused (same weights, no second copy)
        self.acc_dtype = acc_dtype
        self.scale_on_x_max_rows = scale_on_x_max_rows
        self.p_half_prefix = p_half_prefix
        self.slab_half_ksplit = slab_half_ksplit
        # per_branch_kv=True restates hf_model_q40.Transformer instead (hf_model_q40.py:236-372): no shared
        # prompt cache, EVERY position of every batch row lives in that row's Q4_0 cache, the rows of the
        # tokens being processed are used exact (:313-314) and stored quantised (:322-343); a prefill takes
        # B prompt rows and fills B caches.
        self.per_branch_kv = per_branch_kv
        self.args = args
        self.sd = sd
        self.dense = dense
        self.quantize_kv = quantize_kv
        self.n_kv_heads = args.n_heads if args.n_kv_heads is None else args.n_kv_heads
        self.head_dim = args.dim // args.n_heads
        self.freqs_cis = precompute_freqs_cis(self.head_dim, args.max_seq_len + args.max_prompt_seq_len,
                                              args.rope_theta)
        self._dense: Dict[str, torch.Tensor] = {}
        self._codes: Dict[str, Tuple[torch.Tensor, torch.Tensor]] = {}
        if share_dense is not None and share_dense.acc_dtype == acc_dtype:
            self._dense = share_dense._dense
        elif dense:
            for i in range(args.n_layers):
                for name in self.LINEARS:
                    key = f"layers.{i}.{name}"
                    N, K = tuple(sd[key + ".shape"])
                    self._dense[key] = dequantize_q40(sd[key + ".w"], sd[key + ".s"], GROUP_SIZE,
                                                      (K, N), DTYPE).to(acc_dtype)
        if scale_on_x_max_rows > 0:
            assert dense, "the scale-on-x variant keeps the dense matrices for calls with more rows"
            for i in range(args.n_layers):
                for name in self.LINEARS:
                    key = f"layers.{i}.{name}"
                    N, K = tuple(sd[key + ".shape"])
                    # codes [N/64, K, 64] (group-major, ready for a batched product), scales fp16 [K, N/64]
                    codes = unpack_codes(sd[key + ".w"]).view(K, N // GROUP_SIZE, GROUP_SIZE).permute(1, 0, 2).to(acc_dtype).contiguous()
                    self._codes[key] = (codes, sd[key + ".s"].view(K, N // GROUP_SIZE))
        self._out_w = sd["output.weight"].to(acc_dtype)
        self.reset()

    def reset(self):
        a = self.args
        self.kv_codes = {}
        self.prompt_len = 0
        self.prompt_k = [None] * a.n_layers      # fp16 [P, Hkv, D]
        self.prompt_v = [None] * a.n_layers
        # suffix caches hold the DEQUANTISED values of what the reference stores in Q4
        shape = (a.max_batch_size, a.max_seq_len, self.n_kv_heads, self.head_dim)
        self.cache_k = [torch.zeros(shape, dtype=DTYPE) for _ in range(a.n_layers)]
        self.cache_v = [torch.zeros(shape, dtype=DTYPE) for _ in range(a.n_layers)]

    def fork(self, origin: int, curr_batch: int, forks: int):
        """Row copy of the per-branch suffix cache (hf_model_q40_kv_shared.py:282-297)."""
        for i in range(self.args.n_layers):
            for c in (self.cache_k[i], self.cache_v[i]):
                c[curr_batch:curr_batch + forks] = c[origin]

    def _linear(self, key: str, x: torch.Tensor) -> torch.Tensor:
        shp = x.shape
        x2 = x.reshape(-1, shp[-1])
        if self.dense and x2.shape[0] <= self.scale_on_x_max_rows:
            codes, scales = self._codes[key]
            a = (x2[:, :, None] * scales[None]).to(self.acc_dtype)            # fp16 product, rounded to fp16: [M, K, G]
            y = torch.bmm(a.permute(2, 0, 1), codes).permute(1, 0, 2).reshape(x2.shape[0], -1).to(DTYPE)
        elif self.dense and self.slab_half_ksplit is not None:
            W = self._dense[key]
            K, N = W.shape
            ks = int(self.slab_half_ksplit(key, K, N))
            steps = (K + 31) // 32
            per = (steps + ks - 1) // ks * 32                             # rows of a slice: whole 32-row steps
            y = torch.zeros((x2.shape[0], N), dtype=self.acc_dtype)
            for k0 in range(0, K, per):
                y += (x2[:, k0:k0 + per].to(self.acc_dtype) @ W[k0:k0 + per]).to(DTYPE).to(self.acc_dtype)
            y = y.to(DTYPE)
        elif self.dense:
            y = (x2.to(self.acc_dtype) @ self._dense[key]).to(DTYPE)
        else:
            N, K = tuple(self.sd[key + ".shape"])
            y = matmul_q40(x2, self.sd[key + ".w"], self.sd[key + ".s"], (K, N))
        return y.reshape(*shp[:-1], -1)

    def _kv_roundtrip(self, x: torch.Tensor, tag=None) -> torch.Tensor:
        """What later steps see of a stored K/V vector: quantise + dequantise
        (hf_model_q40_kv_shared.py:365-366 then :352-353 on the next step).  `tag`: the packed rows and scales of this call
        are kept in self.kv_codes[tag] (what the reference writes into cache_k / cache_k_s), for tests that copy them."""
        if not self.quantize_kv:
            return x
        w, s = quantize_q40(x, GROUP_SIZE)
        if tag is not None:
            self.kv_codes[tag] = (w, s)
        return dequantize_q40(w, s, GROUP_SIZE, x.shape, DTYPE)

    def forward(self, tokens: torch.Tensor, start_pos: int) -> torch.Tensor:
        """tokens int64 [B,S] -> logits fp16 [B,S,vocab] (hf_model_q40_kv_shared.py:492-510)."""
        a = self.args
        B, S = tokens.shape
        sd = self.sd
        h = F.embedding(tokens, sd["tok_embeddings.weight"]).to(DTYPE)
        freqs = self.freqs_cis[start_pos:start_pos + S]
        H, Hkv, D = a.n_heads, self.n_kv_heads, self.head_dim
        for i in range(a.n_layers):
            p = f"layers.{i}."
            xn = rmsnorm(h, sd[p + "attention_norm.weight"], a.norm_eps)
            xq = self._linear(p + "attention.wq", xn).view(B, S, H, D)
            xk = self._linear(p + "attention.wk", xn).view(B, S, Hkv, D)
            xv = self._linear(p + "attention.wv", xn).view(B, S, Hkv, D)
            xq, xk = apply_rotary_emb(xq, xk, freqs)
            if self.per_branch_kv:
                ck, cv = self.cache_k[i], self.cache_v[i]
                sk = torch.cat((ck[:B, :start_pos], xk), dim=1)
                sv = torch.cat((cv[:B, :start_pos], xv), dim=1)
                ck[:B, start_pos:start_pos + S] = self._kv_roundtrip(xk)
                cv[:B, start_pos:start_pos + S] = self._kv_roundtrip(xv)
                if S == 1:
                    none = torch.zeros((0, Hkv, D), dtype=DTYPE)
                    attn = shared_prefix_attention(xq[:, 0], none, none, sk, sv, [start_pos + 1] * B)[:, None]
                else:
                    assert start_pos == 0, "multi-token calls are prefills"
                    attn = torch.stack([causal_attention(xq[b], xk[b], xv[b], self.acc_dtype, self.p_half_prefix) for b in range(B)])
            elif start_pos == 0:
                # prefill: prompt KV taken from row 0 only, kept in fp16 (:324-329)
                self.prompt_k[i] = xk[0].clone()
                self.prompt_v[i] = xv[0].clone()
                attn = torch.stack([causal_attention(xq[b], xk[b], xv[b], self.acc_dtype, self.p_half_prefix) for b in range(B)])
            else:
                assert S == 1
                t = start_pos - self.prompt_len
                # this step attends to the exact fp16 K/V of the new token (:355-356) ...
                ck, cv = self.cache_k[i], self.cache_v[i]
                sk = torch.cat((ck[:B, :t], xk), dim=1)
                sv = torch.cat((cv[:B, :t], xv), dim=1)
                # ... and later steps see its Q4 round trip (:365-371)
                ck[:B, t] = self._kv_roundtrip(xk[:, 0], (i, "k"))
                cv[:B, t] = self._kv_roundtrip(xv[:, 0], (i, "v"))
                attn = shared_prefix_attention(xq[:, 0], self.prompt_k[i], self.prompt_v[i],
                                               sk, sv, [t + 1] * B, self.acc_dtype, self.p_half_prefix)[:, None]
            attn = attn.reshape(B, S, H * D)
            h = h + self._linear(p + "attention.wo", attn)
            xn = rmsnorm(h, sd[p + "ffn_norm.weight"], a.norm_eps)
            g = self._linear(p + "feed_forward.w1", xn)
            u = self._linear(p + "feed_forward.w3", xn)
            h = h + self._linear(p + "feed_forward.w2", silu_mul(g, u))
        if start_pos == 0 and not self.per_branch_kv:
            self.prompt_len = S
        h = rmsnorm(h, sd["norm.weight"], a.norm_eps)
        return (h.to(self.acc_dtype) @ self._out_w.t()).to(DTYPE)

    def forced(self, prompt: torch.Tensor, tokens: torch.Tensor) -> torch.Tensor:
        """Teacher-forced run of one branch: prefill, then step s is fed tokens[s-1] whatever this model would have
        picked.  Returns the fp32 view of the fp16 logits of every step, [len(tokens), vocab]; row 0 is the prefill's."""
        self.reset()
        P = prompt.shape[1]
        rows = [self.forward(prompt[:1], 0)[0, -1].float()]
        for sidx in range(1, tokens.numel()):
            rows.append(self.forward(tokens[sidx - 1].view(1, 1), P + sidx - 1)[0, -1].float())
        return torch.stack(rows)

    def greedy(self, prompt: torch.Tensor, batch_size: int, steps: int):
        """Prefill once at B=1, fork to `batch_size` branches, greedy decode `steps` tokens
        (argmax, lowest index on ties: hf_model_q40.py:517-519).  Returns (tokens [B,steps],
        margins [steps] = top1-top2 logit gap of branch 0)."""
        self.reset()
        logits = self.forward(prompt[:1], 0)[:, -1].float()
        P = prompt.shape[1]
        out = torch.zeros((batch_size, steps), dtype=torch.int64)
        margins = []
        nxt = logits.argmax(-1).expand(batch_size).clone()
        top2 = logits[0].topk(2).values
        margins.append(float(top2[0] - top2[1]))
        out[:, 0] = nxt
        if batch_size > 1:
            self.fork(0, 1, batch_size - 1)
        for sidx in range(1, steps):
            logits = self.forward(out[:, sidx - 1: sidx], P + sidx - 1)[:, -1].float()
            out[:, sidx] = logits.argmax(-1)
            top2 = logits[0].topk(2).values
            margins.append(float(top2[0] - top2[1]))
        return out, margins


def random_q40_state_dict(args: OracleArgs, seed: int, std: float = 0.02) -> Dict[str, torch.Tensor]:
    """Random-init checkpoint in the converter's output format (fp16_to_int4.py:165-184):
    every linear ~N(0, std) fp16 -> Q4_0 of the transpose; fp16 embeddings and lm_head; unit norms."""
    g = torch.Generator().manual_seed(seed)
    hk = (args.n_heads if args.n_kv_heads is None else args.n_kv_heads) * (args.dim // args.n_heads)
    ffn = ffn_hidden_dim(args.dim, args.multiple_of, args.ffn_dim_multiplier)
    shapes = {"attention.wq": (args.dim, args.dim), "attention.wk": (hk, args.dim),
              "attention.wv": (hk, args.dim), "attention.wo": (args.dim, args.dim),
              "feed_forward.w1": (ffn, args.dim), "feed_forward.w2": (args.dim, ffn),
              "feed_forward.w3": (ffn, args.dim)}
    sd: Dict[str, torch.Tensor] = {}
    sd["tok_embeddings.weight"] = (torch.randn((args.vocab_size, args.dim), generator=g) * std).to(DTYPE)
    sd["output.weight"] = (torch.randn((args.vocab_size, args.dim), generator=g) * std).to(DTYPE)
    sd["norm.weight"] = torch.ones(args.dim, dtype=DTYPE)
    for i in range(args.n_layers):
        p = f"layers.{i}."
        sd[p + "attention_norm.weight"] = torch.ones(args.dim, dtype=DTYPE)
        sd[p + "ffn_norm.weight"] = torch.ones(args.dim, dtype=DTYPE)
        for name, (n, k) in shapes.items():
            v = (torch.randn((n, k), generator=g) * std).to(DTYPE)
            w, s, shp = quantize_weight(v)
            sd[p + name + ".w"], sd[p + name + ".s"], sd[p + name + ".shape"] = w, s, shp
    return sd


# --------------------------------------------------------------------------------------------
# numpy restatement of the codec used to cross-check torch's rounding (independent library)
# --------------------------------------------------------------------------------------------
def np_dequant_table() -> np.ndarray:
    """[16 nibble patterns, 65536 scale bit patterns] -> fp16 bit patterns of nibble*scale,
    computed with numpy float16 arithmetic (nibble pattern p decodes to p-16 if p >= 8)."""
    scales = np.arange(65536, dtype=np.uint16).view(np.float16)
    q = np.array([p - 16 if p >= 8 else p for p in range(16)], dtype=np.float16)
    with np.errstate(all="ignore"):
        return (q[:, None] * scales[None, :]).view(np.uint16)
