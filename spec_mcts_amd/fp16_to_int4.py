"""Checkpoint conversion: HF CodeLlama fp16/bf16 weights -> the Q4_0 `.w/.s/.shape` state dict.

Function form of the reference's conversion script (fp16_to_int4.py:117-201): same key renaming
(HF names -> Meta names), same set of quantised tensors (the seven linears of every layer), same
layout (the TRANSPOSED weight is quantised in groups of 64 along the output dimension), same
output keys.  Embeddings, norms and lm_head stay as loaded.

Two forms: convert_checkpoint quantises on the host, shard by shard, as the reference script does;
convert_checkpoint_streaming walks the shards tensor by tensor (memory-mapped .bin shards or safetensors), quantises each
linear on the GPU with the HIP quantiser and keeps only the 4.25-bit result, so neither the host nor the device ever
holds more than one weight in 16-bit form - what a 70B-class checkpoint needs.  Both give the same bytes.
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


def _is_quantised_key(k: str) -> bool:
    keys = k.split(".")
    return len(keys) == 5 and keys[0] == "layers" and keys[2] in QUANTIZED and keys[3] in QUANTIZED[keys[2]] and keys[4] == "weight"


def iter_checkpoint_tensors(model_dir: str):
    """(Meta-style name, tensor) for every tensor of every shard under model_dir, one at a time.  `pytorch_model-*.bin`
    shards are memory-mapped (tensors only, nothing in the file is executed), `*.safetensors` shards are read tensor by
    tensor; a tensor's bytes leave the disk when it is used."""
    files = sorted(os.listdir(model_dir))
    for file in files:
        path = os.path.join(model_dir, file)
        if file.startswith("pytorch_model-") and file.endswith(".bin"):
            shard = torch.load(path, map_location="cpu", mmap=True, weights_only=True)
            for k in list(shard.keys()):
                (name, v), = remap_state_dict({k: shard.pop(k)}).items()
                yield name, v
        elif file.endswith(".safetensors"):
            from safetensors import safe_open
            with safe_open(path, framework="pt", device="cpu") as f:
                for k in f.keys():
                    (name, v), = remap_state_dict({k: f.get_tensor(k)}).items()
                    yield name, v


def quantize_linear_weight_gpu(v: torch.Tensor, device="cuda:0"):
    """quantize_linear_weight on the GPU: the weight goes to the device in its own dtype, is transposed there and quantised
    by the HIP kernel for that dtype (same bytes as the host quantiser).  Returns device tensors (w, s, shape)."""
    from . import kernels as K
    if v.dim() != 2 or v.shape[0] % 128 != 0:
        raise ValueError(f"out_features must be a multiple of 128, got {tuple(v.shape)}")
    vt = v.to(device).t().contiguous()
    w, s = K.quantize_q40(vt, GROUP_SIZE)
    return w, s, torch.Size(v.shape)


def convert_checkpoint_streaming(model_dir: str, out_file=None, device="cuda:0") -> Dict[str, torch.Tensor]:
    """convert_checkpoint with the GPU quantiser, one tensor at a time; the result (host tensors) is saved to out_file
    when given.  Same keys and bytes as convert_checkpoint."""
    out: Dict[str, torch.Tensor] = {}
    for name, v in iter_checkpoint_tensors(model_dir):
        if _is_quantised_key(name):
            base = name[: -len(".weight")]
            w, s, shape = quantize_linear_weight_gpu(v, device)
            out[base + ".w"], out[base + ".s"], out[base + ".shape"] = w.cpu(), s.cpu(), shape
        else:
            out[name] = v
    if out_file is not None:
        torch.save(out, out_file)
    return out
