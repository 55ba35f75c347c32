"""Host-side Q4_0 format code: the checkpoint quantiser and the layout contract.

This is the offline half of the format (what fp16_to_int4.py of the reference does on the CPU when
a checkpoint is converted); the device kernels only ever see its output.  Written with torch
tensor ops so that it runs on whatever device the tensor lives on and inherits torch's rounding.
"""
from __future__ import annotations

from typing import Tuple

import torch

GROUP_SIZE = 64
DTYPE = torch.float16


def quantize_q40_torch(w: torch.Tensor, group_size: int = GROUP_SIZE) -> Tuple[torch.Tensor, torch.Tensor]:
    """Symmetric int4 quantisation in groups of 64: scale = fp16(absmax/7), code = round(w/scale)
    in [-7,7]; groups 2p / 2p+1 go to the high / low nibbles of packed row p
    (reference: fp16_to_int4.py:52-81).  Returns (int8 [numel/128, 64], fp16 [numel/64, 1])."""
    if group_size != GROUP_SIZE:
        raise ValueError("only group_size 64 is supported")
    if w.numel() % (2 * group_size) != 0:
        raise ValueError("numel must be a multiple of 128")
    g = w.reshape(-1, group_size)
    scale = (g.abs().amax(dim=1) / 7.0).to(DTYPE).unsqueeze(1)
    codes = torch.round(g / scale).to(torch.int8).reshape(-1, 2, group_size)
    packed = (codes[:, 0, :] << 4) | (codes[:, 1, :] & 0x0F)
    return packed.contiguous(), scale


def dequantize_q40_torch(w: torch.Tensor, scale: torch.Tensor, group_size: int, shape, ptdtype=DTYPE) -> torch.Tensor:
    """Sign-extending unpack and one fp16 multiply (reference: fp16_to_int4.py:83-96).  Host-side
    utility for checkpoint inspection; the model never calls it."""
    hi = w >> 4
    lo = (w << 4) >> 4
    q = torch.hstack((hi, lo)).view(-1, group_size)
    return (q * scale.view(-1, 1)).to(ptdtype).reshape(shape)


def quantize_linear_weight(v: torch.Tensor):
    """One HF linear weight v[N_out, K_in] -> (w, s, shape) as stored in the checkpoint: the
    TRANSPOSE is quantised, so a scale group is 64 consecutive outputs at fixed k
    (reference: fp16_to_int4.py:173-176)."""
    if v.dim() != 2 or v.shape[0] % 128 != 0:
        raise ValueError(f"out_features must be a multiple of 128, got {tuple(v.shape)}")
    w, s = quantize_q40_torch(v.t(), GROUP_SIZE)
    return w, s, v.shape
