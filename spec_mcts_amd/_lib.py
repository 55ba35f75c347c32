"""ctypes binding of libsmh.so (the C ABI declared in include/smh.h).

The library is built in-tree by spec_mcts_amd.build.  There is no fallback: if the library is
missing, or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_long, c_size_t, c_void_p

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("SMH_LIB", os.path.join(HERE, "libsmh.so"))

SMH_EPI_NONE, SMH_EPI_RESIDUAL = 0, 1
SMH_KV_NONE, SMH_KV_FP16, SMH_KV_Q40 = 0, 1, 2
SMH_GEMV_MAX_M = 16

_P = c_void_p
# name -> (restype, argtypes); must list every symbol of include/smh.h
SIGNATURES = {
    "smh_version": (c_int, []),
    "smh_last_error_string": (c_char_p, []),
    "smh_q40_dequant": (c_int, [_P, _P, _P, c_long, _P]),
    "smh_q40_quantize": (c_int, [_P, _P, _P, c_long, _P]),
    "smh_q40_quantize_f32": (c_int, [_P, c_int, _P, _P, c_long, _P]),
    "smh_q40_matmul_workspace_bytes": (c_size_t, [c_int, c_int]),
    "smh_q40_gemv": (c_int, [_P, c_int, c_int, c_long, _P, _P, c_int, _P, c_long, c_int, _P, c_long, _P, c_size_t, _P]),
    "smh_q40_gemm": (c_int, [_P, c_int, c_int, c_long, _P, _P, c_int, _P, c_long, c_int, _P, c_long, _P, c_size_t, _P]),
    "smh_q40_matmul": (c_int, [_P, c_int, c_int, c_long, _P, _P, c_int, _P, c_long, c_int, _P, c_long, _P, c_size_t, _P]),
    "smh_q40_matmul_plan": (c_int, [c_int, c_int, c_int, _P]),
    "smh_q40_matmul_plan_tiled": (c_int, [c_int, c_int, c_int, _P]),
    "smh_q40_swiglu_fits": (c_int, [c_int, c_int, c_int]),
    "smh_q40_matmul_tiled_swiglu": (c_int, [_P, c_int, c_int, c_long, _P, _P, c_int, _P, c_long, _P]),
    "smh_q40_matmul_partial": (c_int, [_P, c_int, c_int, c_long, c_int, _P, _P, _P, _P, c_size_t, _P]),
    "smh_q40_tiled_bytes": (c_size_t, [c_int, c_int]),
    "smh_q40_tile": (c_int, [_P, _P, c_int, c_int, _P, c_size_t, _P]),
    "smh_q40_matmul_partial_tiled": (c_int, [_P, c_int, c_int, c_long, c_int, _P, _P, _P, c_size_t, _P]),
    "smh_q40_matmul_partial_tiled_silu": (c_int, [_P, c_int, c_int, c_int, c_int, _P, _P, _P, c_size_t, _P]),
    "smh_partial_residual_sumsq": (c_int, [_P, c_int, c_int, c_int, _P, _P, _P, _P]),
    "smh_q40_norm_in_fits": (c_int, [c_int, c_int, c_int, _P]),
    "smh_q40_matmul_partial_tiled_norm": (c_int, [_P, c_long, _P, _P, c_float, c_int, c_int, c_int, _P, _P, _P, c_size_t, _P]),
    "smh_sample_topk_counts": (c_int, [_P, c_int, c_int, c_long, c_float, c_int, _P, _P, _P, c_int, _P]),
    "smh_tree_fork": (c_int, [_P, c_int, _P, _P, _P, _P, c_int, _P, c_long, c_int, _P, c_long, c_int, _P, _P]),
    "smh_tree_step": (c_int, [_P, c_int, _P, _P, _P, _P, c_int, _P, c_long, _P, _P, c_long, _P, _P, _P, c_int, ctypes.c_int64, _P, _P, _P, _P]),
    "smh_detect_terminal": (c_int, [_P, _P, _P, _P, c_int, ctypes.c_int64, c_int, _P]),
    "smh_partial_reduce": (c_int, [_P, c_int, c_int, c_int, c_int, c_int, _P, c_long, c_int, _P, c_long, _P]),
    "smh_partial_rmsnorm": (c_int, [_P, c_int, c_int, c_int, _P, _P, c_float, _P, _P, _P]),
    "smh_partial_silu_mul": (c_int, [_P, c_int, c_int, c_int, _P, _P]),
    "smh_partial_rope_append_kv": (c_int, [_P, c_int, c_int, c_int, c_int, c_int, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P,
                                           c_int, _P, _P]),
    "smh_rmsnorm": (c_int, [_P, _P, _P, c_int, c_int, c_float, _P]),
    "smh_silu_mul": (c_int, [_P, _P, _P, c_long, _P]),
    "smh_argmax": (c_int, [_P, c_int, c_int, c_long, _P, _P]),
    "smh_sample_topk_rowtemp": (c_int, [_P, c_int, c_int, c_long, _P, c_int, _P, _P, _P, c_int, _P]),
    "smh_gq40_quantize": (c_int, [_P, _P, _P, c_long, _P]),
    "smh_gq40_dequant": (c_int, [_P, _P, _P, c_long, _P]),
    "smh_sample_topk": (c_int, [_P, c_int, c_int, c_long, c_float, c_int, _P, _P, _P]),
    "smh_sample_topk_filter": (c_int, [_P, c_int, c_int, c_long, c_float, c_int, _P, _P, _P]),
    "smh_rope_append_kv": (c_int, [_P, _P, _P, c_int, c_int, c_int, c_int, _P, _P, _P, _P, _P, _P, _P, c_int, _P, _P]),
    "smh_rope": (c_int, [_P, _P, c_int, c_int, c_int, c_int, _P, _P, c_int, _P]),
    "smh_set_step": (c_int, [_P, c_int, c_int, _P]),
    "smh_kv_fork": (c_int, [_P, _P, c_int, c_long, c_long, c_int, c_int, c_int, _P]),
    "smh_f16_linear": (c_int, [_P, c_int, c_int, c_long, _P, c_int, _P, c_long, _P]),
    "smh_embedding": (c_int, [_P, c_int, _P, c_int, c_int, _P, _P]),
    "smh_attn_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "smh_shared_prefix_attn": (c_int, [_P, _P, c_int, c_int, c_int, c_int, _P, _P, c_int, c_int, _P, _P, _P, _P, c_int,
                                       _P, c_int, _P, _P, _P, c_size_t, _P]),
    "smh_shared_prefix_attn_one": (c_int, [_P, _P, c_int, c_int, c_int, c_int, _P, _P, c_int, c_int, _P, _P, _P, _P, c_int,
                                       _P, c_int, _P, _P, _P, c_size_t, _P]),
    "smh_attn_static_scratch_bytes": (c_size_t, []),
    "smh_shared_prefix_attn_static": (c_int, [_P, _P, c_int, c_int, c_int, c_int, _P, _P, c_int, c_int, _P, _P, _P, _P, c_int,
                                              _P, c_int, _P, _P, _P]),
    "smh_prefill_attn": (c_int, [_P, _P, _P, _P, c_int, c_int, c_int, c_int, _P]),
    "smh_attn_qkv_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "smh_shared_prefix_attn_qkv": (c_int, [_P, c_int, _P, c_int, c_int, c_int, c_int, _P, _P, _P, _P, _P, c_int,
                                           _P, _P, _P, _P, c_int, _P, _P, c_int, c_int, _P, c_size_t, _P]),
    "smh_paged_prefix_attn": (c_int, [_P, _P, c_int, c_int, c_int, c_int, _P, _P, c_int, c_long, c_long,
                                      c_int, _P, _P, _P, _P, c_long, c_long, c_long, _P, c_int, c_long, c_int, _P, c_int, _P, _P, c_int,
                                      _P, c_size_t, _P]),
    "smh_page_fork": (c_int, [_P, c_int, c_long, c_int, c_int, c_int, c_int, _P]),
}

_lib = None


class SmhError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """Load libsmh.so and declare every entry point.  Raises if the library has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise SmhError(f"{LIB_PATH} not found: build it with `python -m spec_mcts_amd.build` "
                       "(there is no fallback path)")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(status: int, what: str) -> None:
    if status != 0:
        msg = load().smh_last_error_string().decode()
        raise SmhError(f"{what} failed with status {status}: {msg}")
