"""Checkpoint conversion: HF CodeLlama fp16/bf16 weights -> the Q4_0 `.w/.s/.shape` state dict.

Function form of the reference's conversion script (fp16_to_int4.py:117-201): same key renaming
(HF names -> Meta names), same set of quantised tensors (the seven linears of every layer), same
layout (the TRANSPOSED weight is quantised in groups of 64 along the output dimension), same
output keys.  Embeddings, norms and lm_head stay as loaded.
"""
from __future__ import annotations

import os
from typing import Dict

import torch

from .quant import GROUP_SIZE, quantize_linear_weight

# Meta-style name -> HF name (reference: fp16_to_int4.py:117-130)
nameMap = {"attention_norm": "input_layernorm",
           "ffn_norm": "post_attention_layernorm",
           "feed_forward": "mlp",
           "w1": "gate_proj",
           "w2": "down_proj",
           "w3": "up_proj",
           "attention": "self_attn",
           "wq": "q_proj",
           "wk": "k_proj",
           "wv": "v_proj",
           "wo": "o_proj",
           "norm": "norm",
           "output": "lm_head",
           "tok_embeddings": "embed_tokens"}
nameMap_reverse = {v: k for k, v in nameMap.items()}

QUANTIZED = {"attention": ("wq", "wk", "wv", "wo"), "feed_forward": ("w1", "w2", "w3")}


def remap_state_dict(model_dict: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """Strip the 'model.' prefix and translate HF module names to the Meta names the model uses."""
    out = {}
    for k, v in model_dict.items():
        if k.startswith("model."):
            k = k[len("model."):]
        parts = [nameMap_reverse.get(p, p) for p in k.split(".")]
        out[".".join(parts)] = v
    return out


def remap_names(file: str) -> Dict[str, torch.Tensor]:
    """Load one checkpoint shard (tensors only) and rename its keys."""
    return remap_state_dict(torch.load(file, map_location="cpu", mmap=True, weights_only=True))


def quantize_state_dict(sd: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """Replace `layers.N.attention.w{q,k,v,o}.weight` and `layers.N.feed_forward.w{1,2,3}.weight` by
    `<name>.w`, `<name>.s`, `<name>.shape` (reference: fp16_to_int4.py:165-184)."""
    out: Dict[str, torch.Tensor] = {}
    for k, v in sd.items():
        keys = k.split(".")
        if len(keys) >= 4 and keys[0] == "layers" and keys[2] in QUANTIZED and keys[3] in QUANTIZED[keys[2]]:
            base = ".".join(keys[:4])
            w, s, shape = quantize_linear_weight(v)
            out[base + ".w"], out[base + ".s"], out[base + ".shape"] = w, s, shape
        else:
            out[k] = v
    return out


def convert_checkpoint(model_dir: str, out_file: str) -> Dict[str, torch.Tensor]:
    """Convert every `pytorch_model-*.bin` shard under model_dir and save one flat dict."""
    model_dict: Dict[str, torch.Tensor] = {}
    for file in sorted(os.listdir(model_dir)):
        if file.startswith("pytorch_model-"):
            model_dict.update(quantize_state_dict(remap_names(os.path.join(model_dir, file))))
    torch.save(model_dict, out_file)
    return model_dict
