"""Copies the oracle's KV state into the GPU model, so that a multi-step test can hold EVERY step to the tolerance.

A decode step quantises the new token's K/V to Q4_0; a value that sits on a rounding boundary takes a neighbouring code
in one of two faithful implementations, and from then on their caches differ by one quantisation step in that element.
With the oracle's rows written over the model's after each step, every step starts from identical state and its logits
measure that step's arithmetic alone."""
import torch


def sync_prefix(model, oracle):
    """the prompt K/V the oracle's prefill left (fp16 [P, Hkv, D] per layer) into the model's shared prompt cache"""
    for i, layer in enumerate(model.layers):
        att = layer.attention
        P = oracle.prompt_k[i].shape[0]
        assert att.cache_prompt_len == P
        att.cache_prompt_k[0, :P] = oracle.prompt_k[i].to(att.cache_prompt_k.device)
        att.cache_prompt_v[0, :P] = oracle.prompt_v[i].to(att.cache_prompt_v.device)


def sync_suffix_row(model, oracle, B, t):
    """the Q4_0 rows and scales the oracle's last decode step stored at suffix position t of branches 0..B-1 into the model's
    caches (each branch's own row t, which is where the model appended its own)"""
    p = model.params
    for i, layer in enumerate(model.layers):
        att = layer.attention
        Hkv = att.n_local_kv_heads
        for tag, cache, cache_s in (("k", att.cache_k, att.cache_k_s), ("v", att.cache_v, att.cache_v_s)):
            w, s = oracle.kv_codes[(i, tag)]
            cache.view(p.max_batch_size, p.max_seq_len, Hkv, 64)[:B, t] = w.view(B, Hkv, 64).to(cache.device)
            cache_s.view(p.max_batch_size, p.max_seq_len, Hkv, 2)[:B, t] = s.view(B, Hkv, 2).to(cache_s.device)
