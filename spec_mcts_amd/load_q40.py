"""Loader entry: build the Q4_0 Transformer from a converted checkpoint.

Function form of the reference's load_q40.py:95-146: load_state_dict(strict=False, assign=True)
for embeddings / norms / lm_head, attribute assignment of `.w/.s/.shape` for the seven Q4_0
linears of every layer, then model.to(device, fp16).
"""
from __future__ import annotations

from typing import Dict, Optional, Union

import torch

from .fp16_to_int4 import _is_quantised_key, iter_checkpoint_tensors, quantize_linear_weight_gpu, remap_state_dict
from .hf_model_q40_kv_shared import ModelArgs, Transformer

DTYPE = torch.float16
LINEARS = (("attention", "wq"), ("attention", "wk"), ("attention", "wv"), ("attention", "wo"),
           ("feed_forward", "w1"), ("feed_forward", "w2"), ("feed_forward", "w3"))


def assign_q40(model: Transformer, model_dict: Dict[str, torch.Tensor], device) -> None:
    """layer.<block>.<name>.{w,s,shape} <- checkpoint entries, tensors moved to `device`
    (reference: load_q40.py:115-143)."""
    for i, layer in enumerate(model.layers):
        for block, name in LINEARS:
            key = f"layers.{i}.{block}.{name}"
            lin = getattr(getattr(layer, block), name)
            lin.w = model_dict[key + ".w"].to(device).contiguous()
            lin.s = model_dict[key + ".s"].to(device).contiguous()
            lin.shape = torch.Size(model_dict[key + ".shape"])
            K_in, N_out = lin.shape[1], lin.shape[0]
            if N_out % 128 != 0 or lin.w.numel() != K_in * N_out // 2 or lin.s.numel() != K_in * N_out // 64:
                raise ValueError(f"{key}: tensors do not match shape {tuple(lin.shape)} in the Q4_0 layout")


def load_q40(model_file: Union[str, Dict[str, torch.Tensor]], params: Optional[ModelArgs] = None,
             device: str = "cuda:0", model_cls=None) -> Transformer:
    """model_file: path of a converted checkpoint (torch.save of a flat dict) or the dict itself.
    model_cls: the Transformer to build - hf_model_q40_kv_shared.Transformer (default) or
    hf_model_q40.Transformer, with that module's ModelArgs."""
    if isinstance(model_file, str):
        model_dict = torch.load(model_file, map_location="cpu", mmap=True, weights_only=True)
    else:
        model_dict = model_file
    model_dict = remap_state_dict(model_dict)
    if model_cls is None:
        model_cls = Transformer
    model = model_cls(params) if params is not None else (model_cls(ModelArgs()) if model_cls is Transformer else model_cls(__import__("spec_mcts_amd.hf_model_q40", fromlist=["ModelArgs"]).ModelArgs()))
    plain = {k: v for k, v in model_dict.items() if k.split(".")[-1] not in ("w", "s", "shape")}
    model.load_state_dict(plain, strict=False, assign=True)
    assign_q40(model, model_dict, device)
    model.to(device=device, dtype=DTYPE)
    model.eval()
    return model


def load_hf_q40(model_dir: str, params: Optional[ModelArgs] = None, device: str = "cuda:0", model_cls=None) -> Transformer:
    """Build the Q4_0 model straight from an unconverted HF checkpoint directory (fp16 / bf16 shards): every linear is
    sent to the GPU, quantised there and assigned, one tensor at a time, so the 16-bit weights are never held as a whole
    on the host or on the device (a 70B-class checkpoint is ~140 GB in bf16, ~36 GB as Q4_0).  Equivalent to
    fp16_to_int4.convert_checkpoint followed by load_q40."""
    if model_cls is None:
        model_cls = Transformer
    model = model_cls(params if params is not None else ModelArgs())
    plain: Dict[str, torch.Tensor] = {}
    seen = set()
    for name, v in iter_checkpoint_tensors(model_dir):
        if _is_quantised_key(name):
            _, i, block, lname, _ = name.split(".")
            lin = getattr(getattr(model.layers[int(i)], block), lname)
            lin.w, lin.s, lin.shape = quantize_linear_weight_gpu(v, device)
            seen.add((int(i), block, lname))
        else:
            plain[name] = v.to(device=device, dtype=DTYPE) if v.is_floating_point() else v
    missing = [(i, b, n) for i in range(len(model.layers)) for b, n in LINEARS if (i, b, n) not in seen]
    if missing:
        raise ValueError(f"checkpoint lacks {len(missing)} linear weights, first: layers.{missing[0][0]}.{missing[0][1]}.{missing[0][2]}")
    model.load_state_dict(plain, strict=False, assign=True)
    model.to(device=device, dtype=DTYPE)
    model.eval()
    return model
