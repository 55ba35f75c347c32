"""Drop-in model API of the reference's live Q4_0 CodeLlama model, running on the HIP kernels.

Mirrors hf_model_q40_kv_shared.py of the reference: ModelArgs (:58-72), LinearQ4_0 (:217-250),
Attention with a shared fp16 prompt KV cache plus a per-branch Q4_0 suffix KV cache and fork
(:252-409), FeedForward (:412-436), TransformerBlock (:439-467) and Transformer with
forward(tokens, start_pos), fork, resetSeq, resetTimers, printTimers, generate (:470-613).

Same attribute names (`layers[i].attention.wq.w/.s/.shape`, `tok_embeddings`, `norm`, `output`,
`freqs_cis`, cache_* tensors), same call protocol (first call start_pos == 0 = prefill that stores
the prompt KV from row 0; later calls one token per branch), same cast points.  What differs is
the execution: every operator is a HIP kernel (spec_mcts_amd.kernels); the prompt KV is never
copied or expanded per branch and the Q4_0 suffix is decoded inside the attention kernel instead
of being dequantised to a [B, t, H, D] tensor each step.
"""
from __future__ import annotations

import time
from dataclasses import dataclass
from typing import Optional

import torch
import torch.nn.functional as F
from torch import nn

from . import kernels as K

INIT_DEVICE = "meta"
DTYPE = torch.float16
GROUP_SIZE = 64

# wall-clock accumulators with the reference's names (hf_model_q40_kv_shared.py:17-23).  They are
# only filled when Transformer.profile is True, in which case every section is bracketed by a
# device synchronisation so that the numbers mean something.
COMP_TIME = 0.0
DEQ_TIME = 0.0
QKVO_TIME = 0.0
ATTN_TIME = 0.0
MLP_TIME = 0.0
Q_TIME = 0.0
DQ_TIME = 0.0
PROFILE = False


def _tick() -> float:
    if PROFILE:
        torch.cuda.synchronize()
        return time.time()
    return 0.0


@dataclass
class ModelArgs:
    dim: int = 4096
    n_layers: int = 32
    n_heads: int = 32
    n_kv_heads: Optional[int] = None
    vocab_size: int = 32016
    multiple_of: int = 256  # make SwiGLU hidden layer size multiple of large power of 2
    ffn_dim_multiplier: Optional[float] = None
    norm_eps: float = 1e-5
    rope_theta: float = 1000000.0

    max_batch_size: int = 80
    max_seq_len: int = 256
    max_prompt_seq_len: int = 256


def _cache_device() -> torch.device:
    return torch.device("cuda") if torch.cuda.is_available() else torch.device("cpu")


class RMSNorm(torch.nn.Module):
    def __init__(self, dim: int, eps: float = 1e-6):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim))

    def forward(self, x):
        return K.rmsnorm(x, self.weight, self.eps)


def precompute_freqs_cis(dim: int, end: int, theta: float = 10000.0):
    """complex64 [end, dim/2] rotation table, built on the host exactly as the reference does
    (hf_model_q40_kv_shared.py:137-142); the kernels consume its fp16 cos/sin."""
    freqs = 1.0 / (theta ** (torch.arange(0, dim, 2)[: (dim // 2)].float() / dim))
    t = torch.arange(end, dtype=torch.float32)
    freqs = torch.outer(t, freqs)
    return torch.polar(torch.ones_like(freqs), freqs)


class LinearQ4_0(torch.nn.Module):
    """Q4_0 linear.  `.w` (int8 [K*N/128, 64]), `.s` (fp16 [K*N/64]) and `.shape` are plain
    attributes filled by the loader, exactly as in the reference; after loading `.shape` is the
    checkpoint's (out_features, in_features)."""

    def __init__(self, in_features, out_features, group_size):
        super().__init__()
        self.group_size = group_size
        self.w = torch.zeros((int(in_features * out_features / group_size / 2), group_size), dtype=torch.int8, device="cpu")
        self.s = torch.zeros(int(in_features * out_features / group_size), dtype=DTYPE, device="cpu")
        self.shape = (out_features, in_features)
        self._tiled = None
        self._tiled_key = None
        self._released = False

    def release_checkpoint(self):
        """Keep only the tiled copy of this weight on the device: `.w` and `.s` become empty tensors (`.shape` stays), which
        halves the weight bytes the model holds.  The module still multiplies (forward and the model's fused path read the
        tiled copy); operators that take the checkpoint tensors themselves (matmul_q40, triton_deq_int40) no longer can."""
        assert self.w.is_cuda, "the tiled copy lives on the GPU"
        self.operand(True)
        dev = self.w.device
        self.w = torch.empty((0, self.group_size), dtype=torch.int8, device=dev)
        self.s = torch.empty(0, dtype=DTYPE, device=dev)
        self._released = True

    def operand(self, tiled: bool = True):
        """What matmul_q40_partial takes for this weight: (w, s, N) in the checkpoint layout, or - the default
        on the GPU - its tiled copy, made on first use (before any graph capture) and remade when `.w` / `.s`
        are replaced; after changing them in place call `invalidate()`."""
        if self._released:
            assert tiled, "this linear holds only its tiled copy (release_checkpoint)"
            return self._tiled
        if not tiled or not self.w.is_cuda:
            return (self.w, self.s, self.shape[0])
        key = (self.w.data_ptr(), self.s.data_ptr())
        if self._tiled is None or self._tiled_key != key:
            self._tiled = K.tile_q40(self.w, self.s, self.shape[1], self.shape[0])
            self._tiled_key = key
        return self._tiled

    def invalidate(self):
        self._tiled = None

    def forward(self, x, residual=None):
        shape = x.shape
        x = x.reshape(shape[0] * shape[1], shape[2])
        t0 = _tick()
        if residual is not None:
            residual = residual.reshape(shape[0] * shape[1], -1)
        if self._released:
            result = K.partial_reduce(K.matmul_q40_partial(x.contiguous(), [self._tiled]), residual=residual)
        else:
            result = K.matmul_q40(x, self.w, self.s, (self.shape[1], self.shape[0]), residual=residual)
        if PROFILE:
            global COMP_TIME
            COMP_TIME += _tick() - t0
        return result.view((shape[0], shape[1], -1))


class Attention(nn.Module):
    def __init__(self, args: ModelArgs):
        super().__init__()
        self.args = args
        self.n_kv_heads = args.n_heads if args.n_kv_heads is None else args.n_kv_heads
        assert args.n_heads % self.n_kv_heads == 0
        self.n_local_heads = args.n_heads
        self.n_local_kv_heads = self.n_kv_heads
        self.n_rep = self.n_local_heads // self.n_local_kv_heads
        self.head_dim = args.dim // args.n_heads
        assert self.head_dim == 128, "the attention kernels are written for head_dim 128"

        self.wq = LinearQ4_0(args.dim, args.n_heads * self.head_dim, GROUP_SIZE)
        self.wk = LinearQ4_0(args.dim, self.n_kv_heads * self.head_dim, GROUP_SIZE)
        self.wv = LinearQ4_0(args.dim, self.n_kv_heads * self.head_dim, GROUP_SIZE)
        self.wo = LinearQ4_0(args.n_heads * self.head_dim, args.dim, GROUP_SIZE)

        dev = _cache_device()
        prompt_shape = (1, args.max_prompt_seq_len, self.n_local_kv_heads, self.head_dim)
        self.cache_prompt_k = torch.zeros(prompt_shape, dtype=DTYPE, device=dev)
        self.cache_prompt_v = torch.zeros(prompt_shape, dtype=DTYPE, device=dev)
        self.cache_prompt_len = 0

        # per-branch suffix cache in Q4_0: one 64-byte row + 2 scales per (branch, position, kv head).
        # All-zero bytes and scales decode to 0.0, the state the reference reaches by quantising zeros.
        rows = args.max_batch_size * args.max_seq_len * self.n_local_kv_heads
        self.cache_k = torch.zeros((rows, 64), dtype=torch.int8, device=dev)
        self.cache_k_s = torch.zeros((rows * 2, 1), dtype=DTYPE, device=dev)
        self.cache_v = torch.zeros((rows, 64), dtype=torch.int8, device=dev)
        self.cache_v_s = torch.zeros((rows * 2, 1), dtype=DTYPE, device=dev)

    def fork(self, origin: int, curr_batch: int, forks: int):
        """Copy the suffix KV of branch `origin` to branches curr_batch .. curr_batch+forks-1."""
        B = self.args.max_batch_size
        K.kv_fork(self.cache_k, self.cache_k_s, B, origin, curr_batch, forks)
        K.kv_fork(self.cache_v, self.cache_v_s, B, origin, curr_batch, forks)

    def resetSeq(self):
        """Sets sequence length = 0"""
        self.cache_prompt_len = 0

    def decode_attention(self, q, k, v, t_dev, pages, single_launch):
        """One query per branch over the shared prompt rows, the branch's suffix rows 0 .. *t_dev - 1 (its own, or those its
        page-table row names) and the new token's exact k, v."""
        P = self.cache_prompt_len
        if pages is None:
            return K.shared_prefix_attn(q, self.cache_prompt_k[0], self.cache_prompt_v[0], P, suffix_k=self.cache_k, suffix_v=self.cache_v,
                                        suffix_ks=self.cache_k_s, suffix_vs=self.cache_v_s, Smax=self.args.max_seq_len, lens=t_dev,
                                        lens_stride=0, cur_k=k, cur_v=v, single_launch=single_launch)
        Hkv = self.n_local_kv_heads
        return K.paged_prefix_attn(q, pages, t_dev, self.cache_k.view(-1, Hkv, 64), self.cache_v.view(-1, Hkv, 64),
                                   self.cache_k_s.view(-1, Hkv, 2), self.cache_v_s.view(-1, Hkv, 2),
                                   prefix_k=self.cache_prompt_k[0], prefix_v=self.cache_prompt_v[0], P=P, cur_k=k, cur_v=v,
                                   lens_stride=0, single_launch=single_launch)

    def forward(self, x: torch.Tensor, start_pos: int, freqs_cis, mask, residual=None, step_state=None, pages=None):
        """x [B,S,dim] (already normalised); returns residual + wo(attention) when `residual` is given."""
        bsz, seqlen, _ = x.shape
        global QKVO_TIME, ATTN_TIME
        t0 = _tick()
        xq, xk, xv = self.wq(x), self.wk(x), self.wv(x)
        H, Hkv, D = self.n_local_heads, self.n_local_kv_heads, self.head_dim
        cos, sin = freqs_cis
        if start_pos == 0:
            # prefill: rotate, keep the prompt K/V of row 0 in fp16, causal attention per row
            outs = []
            for b in range(bsz):
                q_b = xq[b].view(seqlen, H, D)
                k_b = xk[b].view(seqlen, Hkv, D)
                v_b = xv[b].view(seqlen, Hkv, D)
                K.rope(q_b, k_b, cos, sin, 0)
                if b == 0:
                    self.cache_prompt_k[0, :seqlen] = k_b
                    self.cache_prompt_v[0, :seqlen] = v_b
                    self.cache_prompt_len = seqlen
                t1 = _tick()
                outs.append(K.prefill_attn(q_b, k_b, v_b).view(seqlen, H * D))
            output = torch.stack(outs)
        else:
            assert seqlen == 1, "decode steps take one token per branch"
            pos_dev, t_dev = step_state
            q_b = xq.view(bsz, H, D)
            k_b = xk.view(bsz, Hkv, D)
            v_b = xv.view(bsz, Hkv, D)
            K.rope_append_kv(q_b, k_b, v_b, cos, sin, pos_dev, self.cache_k, self.cache_k_s,
                             self.cache_v, self.cache_v_s, self.args.max_seq_len, t_dev)
            t1 = _tick()
            output = self.decode_attention(q_b, k_b, v_b, t_dev, pages, False).view(bsz, 1, H * D)
        if PROFILE:
            t2 = _tick()
            QKVO_TIME += t1 - t0
            ATTN_TIME += t2 - t1
        return self.wo(output, residual=residual)


class FeedForward(nn.Module):
    def __init__(self, dim: int, hidden_dim: int, multiple_of: int, ffn_dim_multiplier: Optional[float]):
        super().__init__()
        hidden_dim = int(2 * hidden_dim / 3)
        if ffn_dim_multiplier is not None:
            hidden_dim = int(ffn_dim_multiplier * hidden_dim)
        hidden_dim = multiple_of * ((hidden_dim + multiple_of - 1) // multiple_of)

        self.w1 = LinearQ4_0(dim, hidden_dim, GROUP_SIZE)
        self.w2 = LinearQ4_0(hidden_dim, dim, GROUP_SIZE)
        self.w3 = LinearQ4_0(dim, hidden_dim, GROUP_SIZE)

    def forward(self, x, residual=None):
        global MLP_TIME
        t0 = _tick()
        out = self.w2(K.silu_mul(self.w1(x), self.w3(x)), residual=residual)
        if PROFILE:
            MLP_TIME += _tick() - t0
        return out


class TransformerBlock(nn.Module):
    def __init__(self, layer_id: int, args: ModelArgs):
        super().__init__()
        self.n_heads = args.n_heads
        self.dim = args.dim
        self.head_dim = args.dim // args.n_heads
        self.attention = Attention(args)
        self.feed_forward = FeedForward(dim=args.dim, hidden_dim=4 * args.dim, multiple_of=args.multiple_of,
                                        ffn_dim_multiplier=args.ffn_dim_multiplier)
        self.layer_id = layer_id
        self.attention_norm = RMSNorm(args.dim, eps=args.norm_eps)
        self.ffn_norm = RMSNorm(args.dim, eps=args.norm_eps)

    def forward(self, x, start_pos, freqs_cis, mask, step_state=None, pages=None):
        # the residual adds are fused into the epilogues of wo and w2
        h = self.attention.forward(self.attention_norm(x), start_pos, freqs_cis, mask, residual=x, step_state=step_state, pages=pages)
        return self.feed_forward.forward(self.ffn_norm(h), residual=h)


class Transformer(nn.Module):
    def __init__(self, params: ModelArgs):
        super().__init__()
        self.params = params
        self.vocab_size = params.vocab_size
        self.n_layers = params.n_layers

        self.tok_embeddings = nn.Embedding(params.vocab_size, params.dim, device=INIT_DEVICE)
        self.layers = torch.nn.ModuleList()
        for layer_id in range(params.n_layers):
            self.layers.append(TransformerBlock(layer_id, params))
        self.norm = RMSNorm(params.dim, eps=params.norm_eps)
        self.output = nn.Linear(params.dim, params.vocab_size, bias=False, device=INIT_DEVICE)

        self.freqs_cis = precompute_freqs_cis(self.params.dim // self.params.n_heads,
                                              self.params.max_seq_len + self.params.max_prompt_seq_len,
                                              params.rope_theta)
        self._rope_tables = None      # (cos, sin) fp16 [T, 64] on the device
        self._step_state = None       # int32 [2] on the device: (position, suffix index t)
        self.fused = True             # fused decode-layer launches; False runs module by module
        self.per_branch_kv = False    # True: hf_model_q40's protocol (every position in the branch's own Q4_0 cache)
        self.fused_sampler = True          # generate(): temperature / top-k / draw as one kernel instead of five torch ops
        self.silu_in_matmul = True         # up to 2 rows: w2's launch makes its own SiLU(gate)*up activations
        self.swiglu_in_matmul = True       # 33 .. 128 rows, wide FFN: SiLU(gate) * up inside w1|w3's launch (kernels.matmul_q40_swiglu)
        self.tiled_weights = True          # the fused path streams tiled copies of the weights (LinearQ4_0.operand)
        self.attn_single_launch = True     # up to 16 queries per kv head: prefix slices, suffix passes and the merge in one launch
                                           # (above, the one workgroup that merges a kv head's query tiles takes longer than a launch)
        self.norm_in_matmul = True         # RMSNorm made by the matmul that consumes it (a shorter launch in between) ...
        self.norm_in_max_rows = 2          # ... up to this many rows: at 10 rows the matmul's longer prologue costs more than it saves
        self._norm_in_ok = {}
        self.attn_from_qkv = True          # up to 16 branches the attention takes the wq|wk|wv product itself, in one launch
        self._q40_output = None            # quantize_lm_head(): (w, s, padded vocab) of a Q4_0 vocabulary projection
        self.paged_kv = True               # fork = a copy of page ids: forked branches share their ancestor's suffix rows
        self._page_table = None            # int32 [max_batch_size, max_seq_len]: cache row that holds position j of branch b
        self._forked = False               # a fork happened since the last resetSeq (until then every branch reads its own rows)
        self._rows_written = 0             # suffix rows every live branch has after the last decode step

    # -- helpers -------------------------------------------------------------------------------
    def _tables(self, device):
        if self._rope_tables is None or self._rope_tables[0].device != device:
            fc = self.freqs_cis.to("cpu")
            cos = fc.real.to(DTYPE).contiguous().to(device)    # rounded to fp16 as the reference does (:193-194)
            sin = fc.imag.to(DTYPE).contiguous().to(device)
            self._rope_tables = (cos, sin)
        return self._rope_tables

    def _set_step(self, device, start_pos: int):
        """Publish (position, suffix index) to the device for the decode kernels."""
        if self._step_state is None or self._step_state.device != device:
            self._step_state = torch.zeros(2, dtype=torch.int32, device=device)
        prompt_len = self.layers[0].attention.cache_prompt_len
        K.set_step(self._step_state, start_pos, start_pos - prompt_len)      # a one-thread launch: nothing the host waits for
        return self._step_state[0:1], self._step_state[1:2]

    # -- the hot path ----------------------------------------------------------------------------
    def _forward_impl(self, tokens: torch.Tensor, start_pos: int, step_state):
        """Embedding -> blocks -> final norm -> lm_head.  For decode steps (start_pos != 0) the
        position and suffix index are read by the kernels from `step_state` (device int32), so this
        function issues no host-to-device traffic and can be captured in a HIP graph."""
        if self.fused:
            return self._forward_fused(tokens, start_pos, step_state)
        h = K.embedding(tokens, self.tok_embeddings.weight)
        freqs = self._tables(h.device)
        pages = self._pages(h.device) if start_pos != 0 else None
        for layer in self.layers:
            h = layer(h, start_pos, freqs, None, step_state=step_state, pages=pages)
        h = self.norm(h)
        return self._lm_head(h)

    def _forward_fused(self, tokens: torch.Tensor, start_pos: int, step_state):
        """Same arithmetic as the module-by-module path, with the launches of a layer fused:
        residual+RMSNorm | wq,wk,wv (one launch) | RoPE + Q4_0 KV append | attention | wo |
        residual+RMSNorm | w1,w3 (one launch) | SiLU*up | w2.  Every linear leaves fp32 K-slice
        slabs that the next small kernel adds and rounds to fp16 once, exactly where the
        reference's matmul_q40 rounds."""
        bsz, seqlen = tokens.shape
        M = bsz * seqlen
        p = self.params
        h = K.embedding(tokens, self.tok_embeddings.weight).view(M, p.dim)
        cos, sin = self._tables(h.device)
        pending = None                      # product of the previous layer's w2, not yet added to h
        pages = self._pages(h.device) if start_pos != 0 else None
        for layer in self.layers:
            att, ff = layer.attention, layer.feed_forward
            H, Hkv, D = att.n_local_heads, att.n_local_kv_heads, att.head_dim
            tiled = self.tiled_weights
            qkv_ops = [att.wq.operand(tiled), att.wk.operand(tiled), att.wv.operand(tiled)]
            if pending is not None and self._norm_in(M, p.dim, qkv_ops):
                # RMSNorm made inside the matmul: the launch before it only adds the slabs and leaves sums of squares
                h, sums = K.partial_residual_sumsq(pending, h)
                qkv = K.matmul_q40_partial_norm(h, sums, layer.attention_norm.weight, layer.attention_norm.eps, qkv_ops)
            else:
                h, xn = K.partial_rmsnorm(pending, h, layer.attention_norm.weight, layer.attention_norm.eps)
                qkv = K.matmul_q40_partial(xn, qkv_ops)
            if start_pos == 0:
                xq = K.partial_reduce(qkv, 0, H * D).view(bsz, seqlen, H, D)
                xk = K.partial_reduce(qkv, H * D, Hkv * D).view(bsz, seqlen, Hkv, D)
                xv = K.partial_reduce(qkv, (H + Hkv) * D, Hkv * D).view(bsz, seqlen, Hkv, D)
                outs = []
                for b in range(bsz):
                    K.rope(xq[b], xk[b], cos, sin, 0)
                    if self.per_branch_kv:
                        # hf_model_q40.py:322-343: the rows of this call go into row b's cache as Q4_0
                        assert seqlen <= p.max_seq_len
                        for cache, cache_s, x in ((att.cache_k, att.cache_k_s, xk[b]), (att.cache_v, att.cache_v_s, xv[b])):
                            w, sc = K.q_int40(x.reshape(-1), GROUP_SIZE)
                            cache.view(p.max_batch_size, p.max_seq_len, Hkv, 64)[b, :seqlen] = w.view(seqlen, Hkv, 64)
                            cache_s.view(p.max_batch_size, p.max_seq_len, Hkv, 2)[b, :seqlen] = sc.view(seqlen, Hkv, 2)
                    elif b == 0:
                        att.cache_prompt_k[0, :seqlen] = xk[b]
                        att.cache_prompt_v[0, :seqlen] = xv[b]
                        att.cache_prompt_len = seqlen
                    outs.append(K.prefill_attn(xq[b], xk[b], xv[b]).view(seqlen, H * D))
                o = outs[0] if bsz == 1 else torch.cat(outs, 0)
            else:
                assert seqlen == 1, "decode steps take one token per branch"
                pos_dev, t_dev = step_state
                if self.attn_from_qkv and M <= K.SMH_GEMV_MAX_M and M * (H // Hkv) <= 128 and not self.per_branch_kv:
                    # RoPE and the KV append happen inside the attention kernels (one launch fewer)
                    o = K.shared_prefix_attn_qkv(qkv, H, Hkv, D, cos, sin, pos_dev, att.cache_prompt_k[0], att.cache_prompt_v[0],
                                                 att.cache_prompt_len, att.cache_k, att.cache_k_s, att.cache_v, att.cache_v_s,
                                                 p.max_seq_len, t_dev,
                                                 single_launch=self.attn_single_launch and M * (H // Hkv) <= 16,
                                                 pages=pages).view(M, H * D)
                else:
                    q, k, v = K.partial_rope_append_kv(qkv, H, Hkv, D, cos, sin, pos_dev, att.cache_k, att.cache_k_s,
                                                       att.cache_v, att.cache_v_s, p.max_seq_len, t_dev)
                    o = att.decode_attention(q, k, v, t_dev, pages, self.attn_single_launch and M * (H // Hkv) <= 16).view(M, H * D)
            po = K.matmul_q40_partial(o, [att.wo.operand(tiled)])
            gu_ops = [ff.w1.operand(tiled), ff.w3.operand(tiled)]
            if tiled and self.swiglu_in_matmul and K.swiglu_fits(M, p.dim, ff.w1.shape[0]):
                # 33 .. 128 rows and a wide FFN: SiLU(gate) * up leaves w1|w3's launch as the activations of w2
                h, xn = K.partial_rmsnorm(po, h, layer.ffn_norm.weight, layer.ffn_norm.eps)
                pending = K.matmul_q40_partial(K.matmul_q40_swiglu(xn, gu_ops[0], gu_ops[1]), [ff.w2.operand(True)])
                continue
            if self._norm_in(M, p.dim, gu_ops):
                h, sums = K.partial_residual_sumsq(po, h)
                gu = K.matmul_q40_partial_norm(h, sums, layer.ffn_norm.weight, layer.ffn_norm.eps, gu_ops)
            else:
                h, xn = K.partial_rmsnorm(po, h, layer.ffn_norm.weight, layer.ffn_norm.eps)
                gu = K.matmul_q40_partial(xn, gu_ops)
            if tiled and self.silu_in_matmul and M <= K.SILU_IN_MAX_M and ff.w2.shape[1] % 32 == 0 and ff.w2.w.is_cuda:
                pending = K.matmul_q40_partial_silu(gu, [ff.w2.operand(True)])      # SiLU(gate)*up made inside w2's launch
            else:
                act = K.partial_silu_mul(gu)
                pending = K.matmul_q40_partial(act, [ff.w2.operand(tiled)])
        _, hn = K.partial_rmsnorm(pending, h, self.norm.weight, self.norm.eps, want_h=False)
        return self._lm_head(hn.view(bsz, seqlen, p.dim))

    def quantize_lm_head(self, enable: bool = True):
        """Optional: run the vocabulary projection as a Q4_0 matmul.  The reference keeps `output` in fp16 because its format
        needs out_features % 128 == 0 and the vocabulary has 32016 entries (hf_model_q40_kv_shared.py:484); here the weight is
        zero-padded to the next multiple of 128 rows (32128), quantised like every other linear (the transpose, groups of 64
        along the outputs) and the padded logits are cut off.  69.7 MB instead of 262 MB per step; logits differ from the
        fp16 projection by the quantisation error of the weight, so this is off unless asked for."""
        if not enable:
            self._q40_output = None
            return
        W = self.output.weight
        K._need_gpu(W)
        vocab, dim = W.shape
        padded = (vocab + 127) // 128 * 128
        Wp = torch.zeros((padded, dim), dtype=DTYPE, device=W.device)
        Wp[:vocab] = W.detach().to(DTYPE)
        w, s = K.quantize_q40(Wp.t().contiguous(), GROUP_SIZE)
        self._q40_output = (w, s, padded)

    def _lm_head(self, hn: torch.Tensor) -> torch.Tensor:
        """hn [..., dim] -> logits fp16 [..., vocab]"""
        if self._q40_output is None:
            return K.f16_linear(hn, self.output.weight)
        w, s, padded = self._q40_output
        dim = hn.shape[-1]
        logits = K.matmul_q40(hn.reshape(-1, dim), w, s, (dim, padded))
        return logits.view(hn.shape[:-1] + (padded,))[..., : self.vocab_size]

    def _pages(self, device):
        """The page table the attention kernels read suffix rows through, or None while no branch shares rows."""
        if not (self.paged_kv and self._forked) or self.per_branch_kv:
            return None
        return self._table(device)

    def _table(self, device):
        p = self.params
        if self._page_table is None or self._page_table.device != device:
            self._page_table = torch.arange(p.max_batch_size * p.max_seq_len, dtype=torch.int32, device=device).view(p.max_batch_size, p.max_seq_len)
        return self._page_table

    def _norm_in(self, M: int, Kd: int, ops) -> bool:
        """RMSNorm inside the matmul that follows it: tiled weights, few rows, and rows x K-slice small enough for the
        kernel's LDS (asked of the library once per shape)."""
        if not (self.norm_in_matmul and self.tiled_weights and M <= min(self.norm_in_max_rows, K.SMH_GEMV_MAX_M)
                and isinstance(ops[0], K.TiledQ40)):
            return False
        key = (M, Kd, tuple(t.N for t in ops))
        ok = self._norm_in_ok.get(key)
        if ok is None:
            ok = self._norm_in_ok[key] = K.norm_in_fits(M, Kd, list(key[2]))
        return ok

    @torch.inference_mode()
    def forward(self, tokens: torch.Tensor, start_pos: int):
        _bsz, seqlen = tokens.shape
        K._need_gpu(tokens, self.tok_embeddings.weight)
        step_state = None
        if start_pos != 0:
            t = start_pos - self.layers[0].attention.cache_prompt_len
            assert 0 <= t < self.params.max_seq_len, "suffix cache exhausted"
            assert start_pos < self.freqs_cis.shape[0], "position beyond the rotation table"
            assert _bsz <= self.params.max_batch_size
            step_state = self._set_step(tokens.device, start_pos)
            self._rows_written = t + 1
        else:
            assert seqlen <= self.params.max_prompt_seq_len
            self._rows_written = 0
        return self._forward_impl(tokens, start_pos, step_state)

    def fork(self, origin: int, curr_batch: int, forks: int):
        """Forks the process, such that kv-cache is copied from origin batch number to all the list of new batches.
        With paged_kv (the default) nothing of the cache moves: the new branches' page-table rows take the ids of the
        origin's rows written so far, one small launch for the whole model; later rows go to each branch's own slots."""
        assert 0 <= origin < self.params.max_batch_size and forks >= 0 and 0 <= curr_batch and curr_batch + forks <= self.params.max_batch_size
        if self.paged_kv and not self.per_branch_kv:
            if forks > 0 and self._rows_written > 0:
                K.page_fork(self._table(self.layers[0].attention.cache_k.device), origin, curr_batch, forks, self._rows_written)
                self._forked = True
            return
        for layer in self.layers:
            layer.attention.fork(origin, curr_batch, forks)

    def resetSeq(self):
        """Sets all sequence length = 0"""
        for layer in self.layers:
            layer.attention.resetSeq()
        if self._forked:
            if self._page_table is not None:     # back to every branch reading its own rows; in place: captured graphs hold its address
                n = self._page_table.numel()
                self._page_table.copy_(torch.arange(n, dtype=torch.int32, device=self._page_table.device).view_as(self._page_table))
            self._forked = False
        self._rows_written = 0

    def release_checkpoint_weights(self):
        """Drop every linear's checkpoint-layout tensors once their tiled copies exist (LinearQ4_0.release_checkpoint): the model
        then holds one copy of the weights (3.6 GB less at 7B, 38 GB less at the 70B architecture).  Not in the reference,
        whose kernels read the checkpoint layout; call it when nothing outside the model needs `.w` / `.s`."""
        assert self.tiled_weights, "the model must be running on tiled weights"
        for layer in self.layers:
            a, f = layer.attention, layer.feed_forward
            for lin in (a.wq, a.wk, a.wv, a.wo, f.w1, f.w2, f.w3):
                lin.release_checkpoint()
        torch.cuda.empty_cache()

    def resetTimers(self):
        global COMP_TIME, DEQ_TIME, QKVO_TIME, ATTN_TIME, MLP_TIME, Q_TIME, DQ_TIME
        COMP_TIME, DEQ_TIME, QKVO_TIME, ATTN_TIME, MLP_TIME, Q_TIME, DQ_TIME = 0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0

    def printTimers(self):
        if not PROFILE:
            print("Timers are off (set spec_mcts_amd.hf_model_q40_kv_shared.PROFILE = True to fill them)")
            return
        print("Times: QKVO_TIME, ATTN_TIME, MLP_TIME, Q_TIME, DQ_TIME, DEQ_TIME, COMP_TIME")
        print("Times:", QKVO_TIME, ATTN_TIME, MLP_TIME, Q_TIME, DQ_TIME, DEQ_TIME, COMP_TIME)
        print("Measured Sum: ", QKVO_TIME + ATTN_TIME + MLP_TIME)

    # -- sampling loops ----------------------------------------------------------------------------
    @torch.inference_mode()
    def generate(self, idx, batch_size, max_new_tokens, temperature=1.0, top_k=32, enc=None):
        """Flat-batch sampling loop of the reference (hf_model_q40_kv_shared.py:534-613) with one
        change of execution, not of result: the prompt is prefilled once (B=1) and the branches
        share its KV, instead of prefilling batch_size identical rows.  temperature == 0.0 selects
        greedy decoding (hf_model_q40.py:517-519)."""
        self.resetTimers()
        self.resetSeq()
        assert self.params.max_batch_size >= batch_size
        idx = idx[:1]
        max_new_tokens = min(max_new_tokens, self.params.max_seq_len)
        results = torch.zeros(batch_size, max_new_tokens, dtype=torch.int64, device=idx.device)
        results_len = torch.zeros(batch_size, dtype=torch.int32, device=idx.device)
        results_mask = results_len == 0
        curr_pos = 0
        for num_new_tokens in range(max_new_tokens):
            if curr_pos == 0:
                idx_cond = idx if idx.size(1) <= self.params.max_prompt_seq_len else idx[:, -self.params.max_prompt_seq_len:]
                logits = self(idx_cond, 0)
                curr_pos += idx_cond.shape[1]
                logits = logits[:, -1, :].expand(batch_size, -1)
            else:
                logits = self(results[:, num_new_tokens - 1: num_new_tokens], curr_pos)
                curr_pos += 1
                logits = logits[:, -1, :]
            if temperature == 0.0:
                idx_next = K.argmax(logits.contiguous())[:, None]
            elif self.fused_sampler and logits.dtype == torch.float16 and top_k <= 1024:
                # division, top-k, softmax and the draw in one launch; torch.rand supplies the randomness
                idx_next = K.sample_topk(logits.contiguous(), temperature, top_k)[:, None]
            else:
                logits = logits / temperature
                v, top_k_idx = torch.topk(logits, top_k)
                probs = F.softmax(v, dim=-1)
                sample = torch.multinomial(probs, num_samples=1, replacement=True)
                idx_next = torch.gather(top_k_idx, 1, sample)
            results[:, num_new_tokens] = idx_next[:, 0] * results_mask.int()
            ends = (idx_next[:, 0] == 2)
            results_len += (~ends).int() * results_mask * 1
            results_mask = ~((ends) | ~results_mask)
            if torch.sum(~results_mask) == batch_size:
                return results[:, :num_new_tokens], results_len
        return results, results_len
