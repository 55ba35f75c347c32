"""Drop-in for the reference's hf_model_q40.py: the same Q4_0 transformer with the OLDER KV protocol.

Differences from hf_model_q40_kv_shared (all of them the reference's, hf_model_q40.py:56-69,236-372,
460-478): `ModelArgs` has no max_prompt_seq_len (defaults 64 rows x 512 positions); there is no shared
prompt cache - every position of every batch row lives in that row's own Q4_0 cache, so a prefill takes
[B, S] prompt rows and fills B caches; `forward` returns fp32 logits.  The arithmetic of a layer is the
same, so the kernels are the same: a decode step is the shared-prefix path with an empty prefix.

The reference re-quantises a 64-position window of the cache on every call (:318-343); quantising rows
that already hold quantised values (or zeros) gives the same rows back, so only the rows of the call
are written here.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch
import torch.nn.functional as F

from . import hf_model_q40_kv_shared as shared
from . import kernels as K


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

    max_batch_size: int = 64
    max_seq_len: int = 512


class Transformer(shared.Transformer):
    def __init__(self, params: ModelArgs):
        inner = shared.ModelArgs(dim=params.dim, n_layers=params.n_layers, n_heads=params.n_heads, n_kv_heads=params.n_kv_heads,
                                 vocab_size=params.vocab_size, multiple_of=params.multiple_of,
                                 ffn_dim_multiplier=params.ffn_dim_multiplier, norm_eps=params.norm_eps,
                                 rope_theta=params.rope_theta, max_batch_size=params.max_batch_size,
                                 max_seq_len=params.max_seq_len, max_prompt_seq_len=params.max_seq_len)
        super().__init__(inner)
        self.params = params                       # what callers read back (hf_model_q40.py:437)
        self._inner_params = inner
        self.per_branch_kv = True
        # prefill needs max_prompt_seq_len = max_seq_len positions of RoPE and nothing of the prompt cache
        for layer in self.layers:
            att = layer.attention
            att.cache_prompt_k = att.cache_prompt_k[:, :1].clone()
            att.cache_prompt_v = att.cache_prompt_v[:, :1].clone()

    @torch.inference_mode()
    def forward(self, tokens: torch.Tensor, start_pos: int):
        _bsz, seqlen = tokens.shape
        K._need_gpu(tokens, self.tok_embeddings.weight)
        assert _bsz <= self.params.max_batch_size and start_pos + seqlen <= self.params.max_seq_len
        saved = self.params
        self.params = self._inner_params           # the shared implementation reads max_prompt_seq_len
        try:
            step_state = None
            if start_pos != 0:
                assert seqlen == 1, "decode steps take one token per row (multi-token calls are prefills)"
                step_state = self._set_step(tokens.device, start_pos)
            out = self._forward_impl(tokens, start_pos, step_state)
        finally:
            self.params = saved
        return out.float()                         # hf_model_q40.py:476

    def fork(self, origin: int, curr_batch: int, forks: int):
        raise AttributeError("hf_model_q40.Transformer has no fork (hf_model_q40_kv_shared.Transformer does)")

    @torch.inference_mode()
    def generate(self, idx, batch_size, max_new_tokens, temperature=1.0, top_k=None, enc=None):
        """hf_model_q40.py:480-537: every row prefills the prompt into its own cache, then the flat-batch
        sampling loop; temperature 0.0 is greedy, otherwise optional top-k filtering + multinomial."""
        assert self.params.max_batch_size >= batch_size
        idx = idx.expand(batch_size, -1)
        curr_pos = 0
        max_new_tokens = min(max_new_tokens, self.params.max_seq_len - idx.shape[1])
        results = torch.zeros(batch_size, max_new_tokens, dtype=torch.int64, device=idx.device)
        results_len = torch.zeros(batch_size, dtype=torch.int32, device=idx.device)
        results_mask = results_len == 0
        for num_new_tokens in range(max_new_tokens):
            if curr_pos == 0:
                logits = self(idx.contiguous(), 0)
                curr_pos += idx.shape[1]
            else:
                logits = self(results[:, num_new_tokens - 1: num_new_tokens], curr_pos)
                curr_pos += 1
            logits = logits[:, -1, :]
            if temperature == 0.0:
                idx_next = K.argmax(logits.half().contiguous())[:, None]
            elif self.fused_sampler and top_k is not None and top_k <= 1024:
                # division, top-k filter, softmax and the draw in one launch (the float32 logits are exact copies of fp16
                # values, so the kernel reads those); torch.rand supplies the randomness
                idx_next = K.sample_topk_filter(logits.half().contiguous(), temperature, top_k)[:, None]
            else:
                logits = logits / temperature
                if top_k is not None:
                    v, _ = torch.topk(logits, min(top_k, logits.size(-1)))
                    logits[logits < v[:, [-1]]] = -float("Inf")
                probs = F.softmax(logits, dim=-1)
                idx_next = torch.multinomial(probs, num_samples=1)
            results[:, num_new_tokens] = idx_next[:, 0] * results_mask.int()
            ends = (idx_next[:, 0] == 2)
            results_len += (~ends).int() * results_mask * 1
            results_mask = ~((ends) | ~results_mask)
            if torch.sum(~results_mask) == batch_size:
                return results[:, :num_new_tokens], results_len
        return results, results_len
