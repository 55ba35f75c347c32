"""Operator surface of the MI355X Q4_0 hot path: torch tensors in, torch tensors out, every
operator a call through the C ABI into a hand-written HIP kernel.

The names and argument meaning mirror the reference's operator file (triton_kernels.py):
matmul_q40 (:471), triton_deq_int40 (:93), quantize_q40 (:12), dequantize_q40 (:43).  As there,
inputs are borrowed, outputs are fresh tensors on the input's device, launches are asynchronous on
the current stream and argument errors are assertions.  There is no CPU or eager fallback: tensors
must live on the GPU and the library must be built.
"""
from __future__ import annotations

import math
from typing import Dict, Optional, Sequence, Tuple

import torch

from . import _lib
from ._lib import SMH_EPI_NONE, SMH_EPI_RESIDUAL, SMH_GEMV_MAX_M, SMH_KV_FP16, SMH_KV_NONE, SMH_KV_Q40, check
from .quant import GROUP_SIZE, quantize_q40_torch

DTYPE_torch = torch.float16

_workspaces: Dict[Tuple[str, int], torch.Tensor] = {}


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _need_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        assert t.is_cuda, "spec_mcts_amd kernels need GPU tensors (there is no CPU fallback)"


def matmul_workspace(device: torch.device, max_m: int = 16, max_n: int = 0) -> torch.Tensor:
    """Per-device scratch that carries the fp32 K-slice slabs from the matmul kernel to its reduce
    kernel.  Shared by all calls on the device (calls run in stream order); calls issued on
    different streams at the same time need their own workspace."""
    lib = _lib.load()
    need = lib.smh_q40_matmul_workspace_bytes(int(max_m), int(max_n))
    key = ("matmul", device.index if device.index is not None else torch.cuda.current_device())
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < need:
        ws = torch.empty(need, dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def attn_workspace(device: torch.device, B: int, H: int, P: int) -> torch.Tensor:
    lib = _lib.load()
    need = lib.smh_attn_workspace_bytes(int(B), int(H), int(P))
    key = ("attn", device.index if device.index is not None else torch.cuda.current_device())
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < need:
        ws = torch.empty(need, dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def attn_qkv_workspace(device: torch.device, B: int, H: int, P: int) -> torch.Tensor:
    """Workspace of the one-launch attention: arrival counters (zero between calls) followed by the partials."""
    lib = _lib.load()
    need = lib.smh_attn_qkv_workspace_bytes(int(B), int(H), int(P))
    key = ("attn_qkv", device.index if device.index is not None else torch.cuda.current_device())
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < need:
        ws = torch.zeros(need, dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


# ---------------------------------------------------------------------------------------------
# Q4_0 matmul
# ---------------------------------------------------------------------------------------------
def matmul_q40(a: torch.Tensor, b_w: torch.Tensor, b_s: torch.Tensor, b_shape: Sequence[int],
               residual: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """c[M,N] = a[M,K] . deq(b_w, b_s)[K,N] in fp16 with fp32 accumulation
    (reference: triton_kernels.py:471-500).  `residual` ([M,N] fp16) fuses the block's residual
    add: c = residual + fp16(a . deq)."""
    lib = _lib.load()
    assert a.is_contiguous(), "Matrix A must be contiguous"
    assert a.dtype == torch.float16 and a.dim() == 2
    M, K = a.shape
    K_b, N = int(b_shape[0]), int(b_shape[1])
    assert K == K_b, "Incompatible dimensions"
    _need_gpu(a, b_w, b_s)
    assert b_w.is_contiguous() and b_s.is_contiguous()
    assert b_w.dtype == torch.int8 and b_w.numel() == K * N // 2, "packed weight does not match b_shape"
    assert b_s.dtype == torch.float16 and b_s.numel() == K * N // 64, "scales do not match b_shape"
    assert a.data_ptr() % 16 == 0
    c = out if out is not None else torch.empty((M, N), device=a.device, dtype=DTYPE_torch)
    assert c.shape == (M, N) and c.is_contiguous() and c.dtype == torch.float16
    epi = SMH_EPI_NONE
    if residual is not None:
        assert residual.shape == (M, N) and residual.is_contiguous() and residual.dtype == torch.float16
        epi = SMH_EPI_RESIDUAL
    ws = matmul_workspace(a.device, M, N)
    check(lib.smh_q40_matmul(a.data_ptr(), M, K, K, b_w.data_ptr(), b_s.data_ptr(), N, c.data_ptr(), N,
                             epi, _ptr(residual), N, ws.data_ptr(), ws.numel(), _stream()), "smh_q40_matmul")
    return c


def matmul_plan(M: int, K: int, ns: Sequence[int], tiled: bool = False) -> int:
    """Number of K slices the matmul kernels use for a [M,K] x [K, sum(ns)] product on checkpoint-layout or on tiled
    weights (the same up to 16 rows)."""
    import ctypes
    lib = _lib.load()
    arr = (ctypes.c_int * len(ns))(*[int(n) for n in ns])
    ks = (lib.smh_q40_matmul_plan_tiled if tiled else lib.smh_q40_matmul_plan)(int(M), int(K), len(ns), arr)
    if ks < 1:
        check(ks, "smh_q40_matmul_plan_tiled" if tiled else "smh_q40_matmul_plan")
    return ks


class PartialProduct:
    """fp32 K-slice slabs [ksplit, M, n_total] left by matmul_q40_partial, to be consumed by one of
    the partial_* operators."""
    __slots__ = ("buf", "ksplit", "M", "n_total")

    def __init__(self, buf, ksplit, M, n_total):
        self.buf, self.ksplit, self.M, self.n_total = buf, ksplit, M, n_total


class TiledQ40:
    """A Q4_0 weight [K, N] rewritten into the matmul kernels' tile order (tile_q40)."""
    __slots__ = ("buf", "K", "N")

    def __init__(self, buf: torch.Tensor, K: int, N: int):
        self.buf, self.K, self.N = buf, K, N


def tile_q40(w: torch.Tensor, s: torch.Tensor, K: int, N: int) -> TiledQ40:
    """Checkpoint layout (w int8 [K*N/128, 64], s fp16 [K*N/64]) -> tiled copy for matmul_q40_partial."""
    lib = _lib.load()
    _need_gpu(w, s)
    assert w.is_contiguous() and s.is_contiguous() and w.dtype == torch.int8 and s.dtype == torch.float16
    assert w.numel() == K * N // 2 and s.numel() == K * N // 64, "packed weight does not match [K, N]"
    nbytes = int(lib.smh_q40_tiled_bytes(K, N))
    buf = torch.empty(nbytes, dtype=torch.uint8, device=w.device)
    check(lib.smh_q40_tile(w.data_ptr(), s.data_ptr(), K, N, buf.data_ptr(), nbytes, _stream()), "smh_q40_tile")
    return TiledQ40(buf, K, N)


def matmul_q40_partial(a: torch.Tensor, linears, out: Optional[torch.Tensor] = None) -> PartialProduct:
    """One launch for up to 3 Q4_0 weights that share the input a [M,K]; `linears` is a sequence of
    (w, s, N), or of TiledQ40 (same slabs, bit for bit).  Leaves the un-reduced product; the columns of the
    weights are concatenated."""
    import ctypes
    lib = _lib.load()
    assert a.is_contiguous() and a.dtype == torch.float16 and a.dim() == 2 and a.data_ptr() % 16 == 0
    _need_gpu(a)
    M, Kd = a.shape
    if isinstance(linears[0], TiledQ40):
        assert all(isinstance(t, TiledQ40) and t.K == Kd for t in linears), "tiled and checkpoint-layout weights cannot share a launch"
        ns = [t.N for t in linears]
        ks = matmul_plan(M, Kd, ns, tiled=True)
        n_total = sum(ns)
        need = ks * M * n_total
        if out is None:
            out = torch.empty(need, dtype=torch.float32, device=a.device)
        assert out.dtype == torch.float32 and out.numel() >= need and out.is_contiguous()
        nseg = len(linears)
        tp = (ctypes.c_void_p * nseg)(*[t.buf.data_ptr() for t in linears])
        na = (ctypes.c_int * nseg)(*ns)
        check(lib.smh_q40_matmul_partial_tiled(a.data_ptr(), M, Kd, Kd, nseg, tp, na, out.data_ptr(), out.numel() * 4, _stream()),
              "smh_q40_matmul_partial_tiled")
        return PartialProduct(out, ks, M, n_total)
    ns = [int(n) for (_, _, n) in linears]
    for (w, s, n) in linears:
        _need_gpu(w, s)
        assert w.is_contiguous() and s.is_contiguous() and w.dtype == torch.int8 and s.dtype == torch.float16
        assert w.numel() == Kd * n // 2 and s.numel() == Kd * n // 64, "packed weight does not match [K, N]"
    ks = matmul_plan(M, Kd, ns)
    n_total = sum(ns)
    need = ks * M * n_total
    if out is None:
        out = torch.empty(need, dtype=torch.float32, device=a.device)
    assert out.dtype == torch.float32 and out.numel() >= need and out.is_contiguous()
    nseg = len(linears)
    wp = (ctypes.c_void_p * nseg)(*[w.data_ptr() for (w, _, _) in linears])
    sp = (ctypes.c_void_p * nseg)(*[s.data_ptr() for (_, s, _) in linears])
    na = (ctypes.c_int * nseg)(*ns)
    check(lib.smh_q40_matmul_partial(a.data_ptr(), M, Kd, Kd, nseg, wp, sp, na, out.data_ptr(), out.numel() * 4, _stream()),
          "smh_q40_matmul_partial")
    return PartialProduct(out, ks, M, n_total)


def swiglu_fits(M: int, K: int, n_half: int) -> bool:
    """Is matmul_q40_swiglu the faster way for these dimensions (17 .. 128 rows, a wide gate / up pair)?"""
    return bool(_lib.load().smh_q40_swiglu_fits(int(M), int(K), int(n_half)))


def matmul_q40_swiglu(a: torch.Tensor, gate: "TiledQ40", up: "TiledQ40", out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp16(silu(fp16(a . gate))) * fp16(a . up) in one launch (FeedForward's `F.silu(self.w1(x)) * self.w3(x)`,
    hf_model_q40_kv_shared.py:434) for tiled weights: what partial_silu_mul(matmul_q40_partial(a, [gate, up])) returns, without
    the slabs.  17 <= M <= 128, K a multiple of 64, n_half a multiple of 128 up to 16384."""
    lib = _lib.load()
    assert a.is_contiguous() and a.dtype == torch.float16 and a.dim() == 2 and a.data_ptr() % 16 == 0
    _need_gpu(a)
    M, Kd = a.shape
    assert isinstance(gate, TiledQ40) and isinstance(up, TiledQ40) and gate.K == Kd and up.K == Kd and gate.N == up.N
    if out is None:
        out = torch.empty((M, gate.N), dtype=torch.float16, device=a.device)
    assert out.shape == (M, gate.N) and out.dtype == torch.float16 and out.is_contiguous()
    check(lib.smh_q40_matmul_tiled_swiglu(a.data_ptr(), M, Kd, Kd, gate.buf.data_ptr(), up.buf.data_ptr(), gate.N, out.data_ptr(), gate.N,
                                          _stream()), "smh_q40_matmul_tiled_swiglu")
    return out


SILU_IN_MAX_M = 2


def matmul_q40_partial_silu(gu: PartialProduct, linears, out: Optional[torch.Tensor] = None) -> PartialProduct:
    """matmul_q40_partial(partial_silu_mul(gu), linears) in one launch for at most SILU_IN_MAX_M rows and tiled
    weights: every workgroup makes the activations of its own K-slice from the gate|up slabs.  Same slabs, bit for bit."""
    import ctypes
    lib = _lib.load()
    M, Kd = gu.M, gu.n_total // 2
    assert M <= SILU_IN_MAX_M and gu.buf.dtype == torch.float32
    assert all(isinstance(t, TiledQ40) and t.K == Kd for t in linears), "tiled weights with K = half the gate|up columns"
    ns = [t.N for t in linears]
    ks = matmul_plan(M, Kd, ns, tiled=True)
    n_total = sum(ns)
    need = ks * M * n_total
    if out is None:
        out = torch.empty(need, dtype=torch.float32, device=gu.buf.device)
    assert out.dtype == torch.float32 and out.numel() >= need and out.is_contiguous() and out.data_ptr() != gu.buf.data_ptr()
    nseg = len(linears)
    tp = (ctypes.c_void_p * nseg)(*[t.buf.data_ptr() for t in linears])
    na = (ctypes.c_int * nseg)(*ns)
    check(lib.smh_q40_matmul_partial_tiled_silu(gu.buf.data_ptr(), gu.ksplit, M, Kd, nseg, tp, na, out.data_ptr(), out.numel() * 4,
                                                _stream()), "smh_q40_matmul_partial_tiled_silu")
    return PartialProduct(out, ks, M, n_total)


def norm_in_fits(M: int, Kd: int, ns) -> bool:
    """Can matmul_q40_partial_norm take this shape (M rows x its K-slice next to the weight rings)?"""
    import ctypes
    if M < 1 or M > SMH_GEMV_MAX_M or Kd % 32 != 0:
        return False
    na = (ctypes.c_int * len(ns))(*ns)
    st = _lib.load().smh_q40_norm_in_fits(M, Kd, len(ns), na)
    check(min(st, 0), "smh_q40_norm_in_fits")
    return st == 1


def partial_residual_sumsq(p: PartialProduct, h_in: Optional[torch.Tensor]):
    """h = h_in + fp16(product), sums[m][0..15] = partial sums of squares of h's row m.  Returns (h, sums)."""
    lib = _lib.load()
    M, N = p.M, p.n_total
    if h_in is not None:
        assert h_in.shape == (M, N) and h_in.is_contiguous() and h_in.dtype == torch.float16
    h = torch.empty((M, N), dtype=torch.float16, device=p.buf.device)
    sums = torch.empty((M, 16), dtype=torch.float32, device=p.buf.device)
    check(lib.smh_partial_residual_sumsq(p.buf.data_ptr(), p.ksplit, M, N, _ptr(h_in), h.data_ptr(), sums.data_ptr(), _stream()),
          "smh_partial_residual_sumsq")
    return h, sums


def matmul_q40_partial_norm(h: torch.Tensor, sums: torch.Tensor, weight: torch.Tensor, eps: float, linears,
                            out: Optional[torch.Tensor] = None) -> PartialProduct:
    """matmul_q40_partial(RMSNorm(h) * weight, linears) in one launch for up to 16 rows and tiled weights, given the
    sums of squares partial_residual_sumsq left: every workgroup normalises its own K-slice.  Same slabs, bit for bit,
    as partial_rmsnorm + matmul_q40_partial."""
    import ctypes
    lib = _lib.load()
    M, Kd = h.shape
    assert h.dtype == torch.float16 and h.is_contiguous() and sums.shape == (M, 16) and sums.dtype == torch.float32
    assert weight.numel() == Kd and weight.dtype == torch.float16
    assert all(isinstance(t, TiledQ40) and t.K == Kd for t in linears), "tiled weights with K = the width of h"
    ns = [t.N for t in linears]
    ks = matmul_plan(M, Kd, ns, tiled=True)
    n_total = sum(ns)
    need = ks * M * n_total
    if out is None:
        out = torch.empty(need, dtype=torch.float32, device=h.device)
    assert out.dtype == torch.float32 and out.numel() >= need and out.is_contiguous()
    nseg = len(linears)
    tp = (ctypes.c_void_p * nseg)(*[t.buf.data_ptr() for t in linears])
    na = (ctypes.c_int * nseg)(*ns)
    check(lib.smh_q40_matmul_partial_tiled_norm(h.data_ptr(), Kd, sums.data_ptr(), weight.data_ptr(), float(eps), M, Kd, nseg, tp, na,
                                                out.data_ptr(), out.numel() * 4, _stream()), "smh_q40_matmul_partial_tiled_norm")
    return PartialProduct(out, ks, M, n_total)


def partial_reduce(p: PartialProduct, col0: int = 0, N: Optional[int] = None, residual: Optional[torch.Tensor] = None) -> torch.Tensor:
    lib = _lib.load()
    N = p.n_total - col0 if N is None else N
    c = torch.empty((p.M, N), dtype=torch.float16, device=p.buf.device)
    epi = SMH_EPI_NONE
    if residual is not None:
        assert residual.shape == (p.M, N) and residual.is_contiguous() and residual.dtype == torch.float16
        epi = SMH_EPI_RESIDUAL
    check(lib.smh_partial_reduce(p.buf.data_ptr(), p.ksplit, p.M, p.n_total, col0, N, c.data_ptr(), N, epi, _ptr(residual), N,
                                 _stream()), "smh_partial_reduce")
    return c


def partial_rmsnorm(p: Optional[PartialProduct], h_in: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                    want_h: bool = True):
    """h = h_in + fp16(product) (either may be absent), xn = RMSNorm(h) * weight.  Returns (h, xn)."""
    lib = _lib.load()
    ref = h_in if h_in is not None else None
    if p is not None:
        M, N = p.M, p.n_total
        dev = p.buf.device
    else:
        M, N = ref.shape
        dev = ref.device
    if h_in is not None:
        assert h_in.shape == (M, N) and h_in.is_contiguous() and h_in.dtype == torch.float16
    assert weight.numel() == N and weight.dtype == torch.float16
    h = torch.empty((M, N), dtype=torch.float16, device=dev) if (want_h and p is not None) else None
    xn = torch.empty((M, N), dtype=torch.float16, device=dev)
    check(lib.smh_partial_rmsnorm(p.buf.data_ptr() if p is not None else None, p.ksplit if p is not None else 1, M, N,
                                  _ptr(h_in), weight.data_ptr(), float(eps), _ptr(h), xn.data_ptr(), _stream()),
          "smh_partial_rmsnorm")
    return (h if h is not None else h_in), xn


def partial_silu_mul(p: PartialProduct) -> torch.Tensor:
    lib = _lib.load()
    n_half = p.n_total // 2
    out = torch.empty((p.M, n_half), dtype=torch.float16, device=p.buf.device)
    check(lib.smh_partial_silu_mul(p.buf.data_ptr(), p.ksplit, p.M, n_half, out.data_ptr(), _stream()), "smh_partial_silu_mul")
    return out


def partial_rope_append_kv(p: PartialProduct, H: int, Hkv: int, D: int, cos: torch.Tensor, sin: torch.Tensor,
                           pos_dev: torch.Tensor, cache_k, cache_ks, cache_v, cache_vs, Smax: int, t_dev):
    """q|k|v product -> fp16 q [B,H,D], k, v [B,Hkv,D] with RoPE applied to q and k, plus the Q4_0
    append of k and v into row t_dev[0] of each branch's suffix cache."""
    lib = _lib.load()
    B = p.M
    assert p.n_total == (H + 2 * Hkv) * D
    dev = p.buf.device
    q = torch.empty((B, H, D), dtype=torch.float16, device=dev)
    k = torch.empty((B, Hkv, D), dtype=torch.float16, device=dev)
    v = torch.empty((B, Hkv, D), dtype=torch.float16, device=dev)
    check(lib.smh_partial_rope_append_kv(p.buf.data_ptr(), p.ksplit, B, H, Hkv, D, q.data_ptr(), k.data_ptr(), v.data_ptr(),
                                         cos.data_ptr(), sin.data_ptr(), pos_dev.data_ptr(), _ptr(cache_k), _ptr(cache_ks),
                                         _ptr(cache_v), _ptr(cache_vs), int(Smax), _ptr(t_dev), _stream()),
          "smh_partial_rope_append_kv")
    return q, k, v


# ---------------------------------------------------------------------------------------------
# Q4_0 codec
# ---------------------------------------------------------------------------------------------
def deq_int40(w: torch.Tensor, s: torch.Tensor, group_size: int, shape, ptdtype=DTYPE_torch) -> torch.Tensor:
    """Q4_0 -> fp16, bit-exact nibble*scale (reference: triton_kernels.py:93-107)."""
    lib = _lib.load()
    assert group_size == GROUP_SIZE and ptdtype == torch.float16
    _need_gpu(w, s)
    assert w.is_contiguous() and s.is_contiguous() and w.dtype == torch.int8 and s.dtype == torch.float16
    n_elements = int(math.prod(shape))
    assert n_elements % 128 == 0 and w.numel() == n_elements // 2 and s.numel() == n_elements // 64
    out = torch.empty(n_elements, device=w.device, dtype=torch.float16)
    check(lib.smh_q40_dequant(w.data_ptr(), s.data_ptr(), out.data_ptr(), n_elements // 128, _stream()),
          "smh_q40_dequant")
    return out.view(shape)


def q_int40(w: torch.Tensor, group_size: int = GROUP_SIZE) -> Tuple[torch.Tensor, torch.Tensor]:
    """fp16 -> Q4_0 on the GPU with the rounding of the torch quantiser (round-half-even of the fp16
    quotient), NOT the +0.5-and-truncate of the reference's disabled Triton kernel
    (triton_kernels.py:134)."""
    lib = _lib.load()
    assert group_size == GROUP_SIZE
    _need_gpu(w)
    assert w.dtype == torch.float16
    w = w.contiguous()
    n = w.numel()
    assert n % 128 == 0
    q = torch.empty((n // 128, 64), device=w.device, dtype=torch.int8)
    s = torch.empty((n // 64, 1), device=w.device, dtype=torch.float16)
    check(lib.smh_q40_quantize(w.data_ptr(), q.data_ptr(), s.data_ptr(), n // 64, _stream()), "smh_q40_quantize")
    return q, s


def quantize_gq40(w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """The block-of-32 Q4_0 flavour of the benchmark's first configuration (scale = absmax / 8, q in [0, 15], value =
    (q - 8) * scale; not a format of the reference's code): fp16 [..., K], K % 32 == 0 -> (uint8 [numel/32, 16], fp16 [numel/32])."""
    lib = _lib.load()
    _need_gpu(w)
    assert w.dtype == torch.float16 and w.shape[-1] % 32 == 0
    w = w.contiguous()
    blocks = w.numel() // 32
    packed = torch.empty((blocks, 16), device=w.device, dtype=torch.uint8)
    scale = torch.empty(blocks, device=w.device, dtype=torch.float16)
    check(lib.smh_gq40_quantize(w.data_ptr(), packed.data_ptr(), scale.data_ptr(), blocks, _stream()), "smh_gq40_quantize")
    return packed, scale


def dequantize_gq40(packed: torch.Tensor, scale: torch.Tensor, shape) -> torch.Tensor:
    """Inverse of quantize_gq40: fp16 tensor of `shape`, one fp16 multiply per weight."""
    lib = _lib.load()
    _need_gpu(packed, scale)
    assert packed.dtype == torch.uint8 and packed.is_contiguous() and packed.dim() == 2 and packed.shape[1] == 16
    assert scale.dtype == torch.float16 and scale.is_contiguous() and scale.numel() == packed.shape[0]
    out = torch.empty(tuple(shape), device=packed.device, dtype=torch.float16)
    assert out.numel() == packed.shape[0] * 32
    check(lib.smh_gq40_dequant(packed.data_ptr(), scale.data_ptr(), out.data_ptr(), packed.shape[0], _stream()), "smh_gq40_dequant")
    return out


def linear_gq40(x: torch.Tensor, packed: torch.Tensor, scale: torch.Tensor, shape) -> torch.Tensor:
    """y = x . W^T for W [N, K] held in the block-of-32 flavour: dequantise, then the fp16 linear kernel (fp32 sums, one rounding)."""
    return f16_linear(x, dequantize_gq40(packed, scale, shape))


def q_int40_wide(w: torch.Tensor, group_size: int = GROUP_SIZE) -> Tuple[torch.Tensor, torch.Tensor]:
    """bfloat16 or fp32 -> Q4_0 on the GPU with the roundings torch's CPU quantiser has for those types (scale through
    the tensor's own type, quotient in fp32): what converting a bfloat16 HF checkpoint on the host produces."""
    lib = _lib.load()
    assert group_size == GROUP_SIZE
    _need_gpu(w)
    assert w.dtype in (torch.bfloat16, torch.float32)
    wide = w.contiguous().float()
    n = wide.numel()
    assert n % 128 == 0
    q = torch.empty((n // 128, 64), device=w.device, dtype=torch.int8)
    s = torch.empty((n // 64, 1), device=w.device, dtype=torch.float16)
    check(lib.smh_q40_quantize_f32(wide.data_ptr(), int(w.dtype == torch.bfloat16), q.data_ptr(), s.data_ptr(), n // 64, _stream()),
          "smh_q40_quantize_f32")
    return q, s


def quantize_q40(w: torch.Tensor, group_size: int = GROUP_SIZE) -> Tuple[torch.Tensor, torch.Tensor]:
    """reference: triton_kernels.py:12-41.  GPU tensors use the HIP kernels (fp16, or bfloat16 / fp32 with torch's
    roundings for those types); host tensors use the torch formulation."""
    if w.is_cuda and w.dtype == torch.float16:
        return q_int40(w, group_size)
    if w.is_cuda and w.dtype in (torch.bfloat16, torch.float32):
        return q_int40_wide(w, group_size)
    return quantize_q40_torch(w, group_size)


dequantize_q40 = deq_int40
triton_deq_int40 = deq_int40      # the reference's name for the same operator
triton_q_int40 = q_int40


# ---------------------------------------------------------------------------------------------
# small fused ops
# ---------------------------------------------------------------------------------------------
def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    lib = _lib.load()
    _need_gpu(x, weight)
    assert x.is_contiguous() and x.dtype == torch.float16 and weight.dtype == torch.float16
    dim = x.shape[-1]
    assert weight.numel() == dim
    out = torch.empty_like(x)
    check(lib.smh_rmsnorm(x.data_ptr(), weight.data_ptr(), out.data_ptr(), x.numel() // dim, dim, float(eps),
                          _stream()), "smh_rmsnorm")
    return out


def silu_mul(g: torch.Tensor, u: torch.Tensor) -> torch.Tensor:
    lib = _lib.load()
    _need_gpu(g, u)
    assert g.shape == u.shape and g.is_contiguous() and u.is_contiguous()
    assert g.dtype == torch.float16 and u.dtype == torch.float16
    out = torch.empty_like(g)
    check(lib.smh_silu_mul(g.data_ptr(), u.data_ptr(), out.data_ptr(), g.numel(), _stream()), "smh_silu_mul")
    return out


def argmax(logits: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Greedy pick over the last dim of fp16 logits [rows, vocab]; lowest index on ties.  `out`: int64, `rows`
    contiguous elements to write into (a decode loop's token buffer) instead of a fresh tensor."""
    lib = _lib.load()
    _need_gpu(logits)
    assert logits.dim() == 2 and logits.dtype == torch.float16 and logits.stride(1) == 1
    rows, vocab = logits.shape
    if out is None:
        out = torch.empty(rows, device=logits.device, dtype=torch.int64)
    assert out.dtype == torch.int64 and out.numel() == rows and out.is_contiguous() and out.device == logits.device
    check(lib.smh_argmax(logits.data_ptr(), rows, vocab, logits.stride(0), out.data_ptr(), _stream()), "smh_argmax")
    return out


def sample_topk(logits: torch.Tensor, temperature: float, top_k: int, uniform: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One token per row of fp16 logits [rows, vocab]: top-k of logits / temperature, softmax, one draw (the sampling
    lines of the reference's generate).  `uniform`: fp32 [rows] in [0, 1), default torch.rand on the logits' device."""
    lib = _lib.load()
    _need_gpu(logits)
    assert logits.dim() == 2 and logits.dtype == torch.float16 and logits.stride(1) == 1
    rows, vocab = logits.shape
    if uniform is None:
        uniform = torch.rand(rows, device=logits.device, dtype=torch.float32)
    _need_gpu(uniform)
    assert uniform.dtype == torch.float32 and uniform.numel() == rows and uniform.is_contiguous()
    out = torch.empty(rows, device=logits.device, dtype=torch.int64)
    check(lib.smh_sample_topk(logits.data_ptr(), rows, vocab, logits.stride(0), float(temperature), int(min(top_k, vocab)),
                              uniform.data_ptr(), out.data_ptr(), _stream()), "smh_sample_topk")
    return out


def sample_topk_filter(logits: torch.Tensor, temperature: float, top_k: int, uniform: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One token per row as the flat-cache model's generate draws it (hf_model_q40.py:521-533): float32 logits / temperature,
    values below the top_k-th largest masked (values EQUAL to it all stay), float32 softmax, one draw.  logits: the fp16
    values [rows, vocab] (that model's float32 logits are exact copies of them).  `uniform` as in sample_topk."""
    lib = _lib.load()
    _need_gpu(logits)
    assert logits.dim() == 2 and logits.dtype == torch.float16 and logits.stride(1) == 1
    rows, vocab = logits.shape
    if uniform is None:
        uniform = torch.rand(rows, device=logits.device, dtype=torch.float32)
    _need_gpu(uniform)
    assert uniform.dtype == torch.float32 and uniform.numel() == rows and uniform.is_contiguous()
    out = torch.empty(rows, device=logits.device, dtype=torch.int64)
    check(lib.smh_sample_topk_filter(logits.data_ptr(), rows, vocab, logits.stride(0), float(temperature), int(min(top_k, vocab)),
                                     uniform.data_ptr(), out.data_ptr(), _stream()), "smh_sample_topk_filter")
    return out


def sample_topk_counts(logits: torch.Tensor, temperature, top_k: int, counts: torch.Tensor, uniform: torch.Tensor,
                       out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """sample_topk with counts[r] draws for row r (torch.multinomial(probs[r], num_samples=counts[r], replacement=True) of
    the tree sampler, mcts.py:128): int64 [uniform.numel()] with row r's tokens at counts[:r].sum() onwards.  counts int32
    [rows] and uniform fp32 [>= counts.sum()] on the device.  temperature: a positive number (logits / temperature stays
    fp16, as in torch) or a float32 tensor [rows] of positive numbers on the device (the sampler's per-branch ramp,
    mcts.py:110-114: a tensor divisor promotes to fp32, so quotients and probabilities are fp32)."""
    lib = _lib.load()
    _need_gpu(logits, counts, uniform)
    assert logits.dim() == 2 and logits.dtype == torch.float16 and logits.stride(1) == 1
    rows, vocab = logits.shape
    assert counts.dtype == torch.int32 and counts.is_contiguous() and counts.numel() >= rows
    assert uniform.dtype == torch.float32 and uniform.is_contiguous()
    if out is None:
        out = torch.zeros(uniform.numel(), device=logits.device, dtype=torch.int64)
    assert out.dtype == torch.int64 and out.is_contiguous() and out.numel() >= uniform.numel()
    if isinstance(temperature, torch.Tensor):
        _need_gpu(temperature)
        assert temperature.dtype == torch.float32 and temperature.is_contiguous() and temperature.numel() >= rows
        check(lib.smh_sample_topk_rowtemp(logits.data_ptr(), rows, vocab, logits.stride(0), temperature.data_ptr(), int(min(top_k, vocab)),
                                          uniform.data_ptr(), counts.data_ptr(), out.data_ptr(), uniform.numel(), _stream()), "smh_sample_topk_rowtemp")
        return out
    check(lib.smh_sample_topk_counts(logits.data_ptr(), rows, vocab, logits.stride(0), float(temperature), int(min(top_k, vocab)),
                                     uniform.data_ptr(), counts.data_ptr(), out.data_ptr(), uniform.numel(), _stream()), "smh_sample_topk_counts")
    return out


def tree_fork(draws: torch.Tensor, output_counts: torch.Tensor, alive: torch.Tensor, curr_b: torch.Tensor, results: torch.Tensor, t: int,
              pages: Optional[torch.Tensor] = None, n_rows: int = 0, origin: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One expansion step of the tree sampler's bookkeeping (mcts.py:127-152) on the device, in place: output_counts int32
    [2, batch] (tokens, multiplicities), alive bool/uint8 [batch], curr_b int32 [1], results int64 [batch, steps], pages int32
    [batch, stride] or None.  Returns origin int32 [batch] (-1, or the branch a row was forked from in this call)."""
    lib = _lib.load()
    _need_gpu(draws, output_counts, alive, curr_b, results)
    batch = results.shape[0]
    assert output_counts.dtype == torch.int32 and output_counts.shape == (2, batch) and output_counts.is_contiguous()
    assert draws.dtype == torch.int64 and draws.is_contiguous()
    assert alive.numel() == batch and alive.is_contiguous() and alive.element_size() == 1
    assert curr_b.dtype == torch.int32 and curr_b.numel() == 1
    assert results.dtype == torch.int64 and results.dim() == 2 and results.is_contiguous()
    if pages is not None:
        assert pages.is_cuda and pages.dtype == torch.int32 and pages.dim() == 2 and pages.is_contiguous() and pages.shape[0] >= batch
    if origin is None:
        origin = torch.empty(batch, dtype=torch.int32, device=results.device)
    check(lib.smh_tree_fork(draws.data_ptr(), draws.numel(), output_counts[0].data_ptr(), output_counts[1].data_ptr(), alive.data_ptr(), curr_b.data_ptr(),
                            batch, results.data_ptr(), results.shape[1], int(t), _ptr(pages), pages.shape[1] if pages is not None else 0,
                            int(n_rows), origin.data_ptr(), _stream()), "smh_tree_fork")
    return origin


def tree_step(draws: torch.Tensor, output_counts: torch.Tensor, alive: torch.Tensor, curr_b: torch.Tensor, results: torch.Tensor,
              t_dev: torch.Tensor, pages: Optional[torch.Tensor], origin: torch.Tensor, state: torch.Tensor, terminal_seq: torch.Tensor,
              results_len: torch.Tensor, next_tokens: torch.Tensor, summary: torch.Tensor, eos: int = 2) -> None:
    """One whole step of the tree sampler after the draws (mcts.py:127-175) in one launch, everything in place and the step
    index read from the device (t_dev int32 [1]: the column of `results` and the suffix rows written so far), so that the
    launch can sit in a captured graph: tree_fork, then detect_terminal on the step's column, results_len += alive,
    alive &= ~ended, next_tokens = results[:, t], summary = (branches, ended rows).  alive is uint8 [batch]."""
    lib = _lib.load()
    _need_gpu(draws, output_counts, alive, curr_b, results, t_dev, origin, state, terminal_seq, results_len, next_tokens, summary)
    B, ld = results.shape
    assert draws.dtype == torch.int64 and draws.is_contiguous()
    assert output_counts.dtype == torch.int32 and output_counts.shape == (2, B) and output_counts.is_contiguous()
    assert alive.dtype == torch.uint8 and alive.numel() == B and alive.is_contiguous()
    assert curr_b.dtype == torch.int32 and t_dev.dtype == torch.int32 and summary.dtype == torch.int32 and summary.numel() >= 2
    assert results.dtype == torch.int64 and results.is_contiguous()
    assert origin.dtype == torch.int32 and origin.numel() >= B and state.dtype == torch.int32 and state.numel() == B
    assert results_len.dtype == torch.int32 and results_len.numel() == B and next_tokens.dtype == torch.int64 and next_tokens.numel() >= B
    assert terminal_seq.dtype == torch.int64 and terminal_seq.is_contiguous()
    if pages is not None:
        _need_gpu(pages)
        assert pages.dtype == torch.int32 and pages.dim() == 2 and pages.shape[0] >= B and pages.stride(1) == 1
    check(lib.smh_tree_step(draws.data_ptr(), draws.numel(), output_counts[0].data_ptr(), output_counts[1].data_ptr(), alive.data_ptr(),
                            curr_b.data_ptr(), B, results.data_ptr(), ld, t_dev.data_ptr(), _ptr(pages), pages.stride(0) if pages is not None else 0,
                            origin.data_ptr(), state.data_ptr(), terminal_seq.data_ptr(), terminal_seq.numel(), int(eos), results_len.data_ptr(),
                            next_tokens.data_ptr(), summary.data_ptr(), _stream()), "smh_tree_step")


def detect_terminal(token: torch.Tensor, state: torch.Tensor, terminal_seq: torch.Tensor, eos: int = 2):
    """detectTerminal of the reference's tree sampler (mcts.py:14-28) on the device in one launch.
    token int64 [B], state int32 [B], terminal_seq int64 [L] -> (end bool [B], state int32 [B]); `state` is not modified."""
    lib = _lib.load()
    _need_gpu(token, state, terminal_seq)
    assert token.dtype == torch.int64 and token.dim() == 1 and token.is_contiguous()
    assert state.shape == token.shape and state.dtype == torch.int32
    assert terminal_seq.dtype == torch.int64 and terminal_seq.dim() == 1 and terminal_seq.is_contiguous() and terminal_seq.numel() >= 1
    new_state = state.clone()
    end = torch.empty(token.shape, dtype=torch.uint8, device=token.device)
    check(lib.smh_detect_terminal(token.data_ptr(), new_state.data_ptr(), end.data_ptr(), terminal_seq.data_ptr(),
                                  terminal_seq.numel(), int(eos), token.numel(), _stream()), "smh_detect_terminal")
    return end.view(torch.bool), new_state


def rope(q: torch.Tensor, k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, pos0: int) -> None:
    """In-place rotate-half RoPE of q [S,H,128] and k [S,Hkv,128]; token s is at position pos0+s."""
    lib = _lib.load()
    _need_gpu(q, k, cos, sin)
    assert q.is_contiguous() and k.is_contiguous() and q.dtype == torch.float16 and k.dtype == torch.float16
    S, H, D = q.shape
    assert k.shape[0] == S and k.shape[2] == D and cos.shape[1] == D // 2 and pos0 + S <= cos.shape[0]
    assert cos.dtype == torch.float16 and sin.dtype == torch.float16 and cos.is_contiguous() and sin.is_contiguous()
    check(lib.smh_rope(q.data_ptr(), k.data_ptr(), S, H, k.shape[1], D, cos.data_ptr(), sin.data_ptr(), int(pos0),
                       _stream()), "smh_rope")


def rope_append_kv(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                   pos_dev: torch.Tensor, cache_k: Optional[torch.Tensor], cache_ks: Optional[torch.Tensor],
                   cache_v: Optional[torch.Tensor], cache_vs: Optional[torch.Tensor], Smax: int,
                   t_dev: Optional[torch.Tensor]) -> None:
    """Decode-step RoPE of q [B,H,128], k [B,Hkv,128] at position pos_dev[0] (int32 on the device),
    then Q4_0 append of the rotated k and of v into row t_dev[0] of every branch's suffix cache."""
    lib = _lib.load()
    _need_gpu(q, k, v, pos_dev)
    assert q.is_contiguous() and k.is_contiguous() and v.is_contiguous()
    assert q.dtype == torch.float16 and k.dtype == torch.float16 and v.dtype == torch.float16
    assert pos_dev.dtype == torch.int32 and (t_dev is None or t_dev.dtype == torch.int32)
    B, H, D = q.shape
    check(lib.smh_rope_append_kv(q.data_ptr(), k.data_ptr(), v.data_ptr(), B, H, k.shape[1], D,
                                 cos.data_ptr(), sin.data_ptr(), pos_dev.data_ptr(),
                                 _ptr(cache_k), _ptr(cache_ks), _ptr(cache_v), _ptr(cache_vs), int(Smax), _ptr(t_dev),
                                 _stream()), "smh_rope_append_kv")


def set_step(state: torch.Tensor, pos: int, t: int) -> None:
    """state[0] = pos, state[1] = t on the device, asynchronously (the values are kernel arguments)."""
    _need_gpu(state)
    assert state.dtype == torch.int32 and state.numel() >= 2 and state.is_contiguous()
    check(_lib.load().smh_set_step(state.data_ptr(), int(pos), int(t), _stream()), "smh_set_step")


def kv_fork(cache: torch.Tensor, cache_s: torch.Tensor, Bmax: int, origin: int, curr: int, forks: int) -> None:
    """Copy branch `origin`'s Q4_0 cache rows to branches curr..curr+forks-1."""
    lib = _lib.load()
    _need_gpu(cache, cache_s)
    assert cache.is_contiguous() and cache_s.is_contiguous()
    row_bytes = cache.numel() * cache.element_size() // Bmax
    row_scales = cache_s.numel() // Bmax
    check(lib.smh_kv_fork(cache.data_ptr(), cache_s.data_ptr(), Bmax, row_bytes, row_scales, origin, curr, forks,
                          _stream()), "smh_kv_fork")


# ---------------------------------------------------------------------------------------------
# fp16 vocabulary projection, embedding
# ---------------------------------------------------------------------------------------------
def f16_linear(x: torch.Tensor, weight: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [..., K] . weight [N, K]^T -> [..., N] fp16 (fp32 accumulation, one rounding): nn.Linear without bias, as the
    reference's lm_head (hf_model_q40_kv_shared.py:484,509)."""
    lib = _lib.load()
    _need_gpu(x, weight)
    assert x.dtype == torch.float16 and weight.dtype == torch.float16 and weight.dim() == 2 and weight.is_contiguous()
    N, Kd = weight.shape
    assert x.shape[-1] == Kd and x.is_contiguous()
    M = x.numel() // Kd
    if out is None:
        out = torch.empty(x.shape[:-1] + (N,), dtype=torch.float16, device=x.device)
    assert out.dtype == torch.float16 and out.is_contiguous() and out.numel() == M * N
    check(lib.smh_f16_linear(x.data_ptr(), M, Kd, Kd, weight.data_ptr(), N, out.data_ptr(), N, _stream()), "smh_f16_linear")
    return out


def embedding(tokens: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """table[tokens]: int64 tokens [...] -> fp16 [..., dim] (nn.Embedding of the reference, hf_model_q40_kv_shared.py:477,495)."""
    lib = _lib.load()
    _need_gpu(tokens, table)
    assert tokens.dtype == torch.int64 and table.dtype == torch.float16 and table.dim() == 2 and table.is_contiguous()
    tokens = tokens.contiguous()
    vocab, dim = table.shape
    out = torch.empty(tokens.shape + (dim,), dtype=torch.float16, device=table.device)
    check(lib.smh_embedding(tokens.data_ptr(), tokens.numel(), table.data_ptr(), vocab, dim, out.data_ptr(), _stream()), "smh_embedding")
    return out


# ---------------------------------------------------------------------------------------------
# attention
# ---------------------------------------------------------------------------------------------
def shared_prefix_attn(q: torch.Tensor, prefix_k: Optional[torch.Tensor], prefix_v: Optional[torch.Tensor], P: int,
                       suffix_k: Optional[torch.Tensor] = None, suffix_v: Optional[torch.Tensor] = None,
                       suffix_ks: Optional[torch.Tensor] = None, suffix_vs: Optional[torch.Tensor] = None,
                       Smax: int = 0, lens: Optional[torch.Tensor] = None, lens_stride: int = 1,
                       cur_k: Optional[torch.Tensor] = None, cur_v: Optional[torch.Tensor] = None,
                       n_kv_heads: Optional[int] = None, single_launch: bool = False, out: Optional[torch.Tensor] = None,
                       static_scratch: bool = False) -> torch.Tensor:
    """out[b,h] = softmax(q[b,h] . K_b^T / sqrt(D)) . V_b with K_b = prefix[:P] (shared) ||
    suffix[b, :lens[b]] || cur_k[b].  The suffix is fp16 [B,Smax,Hkv,D] or Q4_0 (int8 rows +
    fp16 scales, the model's cache layout); `lens` is int32 on the device.
    single_launch: one launch instead of two (at most 128 queries per kv head; same result up to fp32
    summation order).  static_scratch: the two-launch form on the library's own static scratch array: with `out`
    given the call allocates nothing (smh_shared_prefix_attn_static)."""
    lib = _lib.load()
    _need_gpu(q)
    assert q.is_contiguous() and q.dtype == torch.float16 and q.dim() == 3
    B, H, D = q.shape
    if prefix_k is not None:
        assert prefix_k.is_contiguous() and prefix_v.is_contiguous() and prefix_k.dtype == torch.float16
        Hkv = prefix_k.shape[-2]
        assert P <= prefix_k.shape[-3]
    else:
        assert P == 0
        Hkv = n_kv_heads if n_kv_heads is not None else (cur_k.shape[1] if cur_k is not None else H)
    fmt = SMH_KV_NONE
    if suffix_k is not None:
        assert suffix_k.is_contiguous() and suffix_v.is_contiguous() and lens is not None
        assert lens.is_cuda and lens.dtype == torch.int32
        if suffix_k.dtype == torch.float16:
            fmt = SMH_KV_FP16
        else:
            assert suffix_k.dtype == torch.int8 and suffix_ks is not None and suffix_vs is not None
            assert suffix_ks.dtype == torch.float16 and suffix_vs.dtype == torch.float16
            fmt = SMH_KV_Q40
    if cur_k is not None:
        assert cur_k.is_contiguous() and cur_v.is_contiguous() and cur_k.dtype == torch.float16
    if out is None:
        out = torch.empty_like(q)
    assert out.shape == q.shape and out.dtype == torch.float16 and out.is_contiguous() and out.device == q.device
    if static_scratch:
        check(lib.smh_shared_prefix_attn_static(q.data_ptr(), out.data_ptr(), B, H, Hkv, D, _ptr(prefix_k), _ptr(prefix_v), int(P),
                                                fmt, _ptr(suffix_k), _ptr(suffix_v), _ptr(suffix_ks), _ptr(suffix_vs), int(Smax),
                                                _ptr(lens), int(lens_stride), _ptr(cur_k), _ptr(cur_v), _stream()),
              "smh_shared_prefix_attn_static")
        return out
    one = bool(single_launch) and B * (H // Hkv) <= 128
    ws = attn_qkv_workspace(q.device, B, H, P) if one else attn_workspace(q.device, B, H, P)
    fn = lib.smh_shared_prefix_attn_one if one else lib.smh_shared_prefix_attn
    check(fn(q.data_ptr(), out.data_ptr(), B, H, Hkv, D, _ptr(prefix_k), _ptr(prefix_v), int(P),
             fmt, _ptr(suffix_k), _ptr(suffix_v), _ptr(suffix_ks), _ptr(suffix_vs), int(Smax),
             _ptr(lens), int(lens_stride), _ptr(cur_k), _ptr(cur_v),
             ws.data_ptr(), ws.numel(), _stream()), "smh_shared_prefix_attn")
    return out


def shared_prefix_attn_qkv(p: PartialProduct, H: int, Hkv: int, D: int, cos: torch.Tensor, sin: torch.Tensor,
                           pos_dev: torch.Tensor, prefix_k: Optional[torch.Tensor], prefix_v: Optional[torch.Tensor], P: int,
                           cache_k: torch.Tensor, cache_ks: torch.Tensor, cache_v: torch.Tensor, cache_vs: torch.Tensor,
                           Smax: int, t_dev: torch.Tensor, single_launch: bool = True,
                           pages: Optional[torch.Tensor] = None) -> torch.Tensor:
    """partial_rope_append_kv + shared_prefix_attn without the RoPE launch and without q/k/v tensors, for up to
    16 branches: the q|k|v product `p` goes straight into the attention kernels.  Returns out [B,H,D].
    single_launch: everything in one launch (the workgroup that finishes last merges); otherwise two launches
    whose result is bit-identical to the separate operators.  pages: int32 [>= B, >= Smax] page table (suffix row j of
    branch b is cache row pages[b, j]); None = every branch reads its own rows."""
    lib = _lib.load()
    B = p.M
    if pages is not None:
        assert pages.is_cuda and pages.dtype == torch.int32 and pages.dim() == 2 and pages.stride(1) == 1
        assert pages.shape[0] >= B and pages.shape[1] >= Smax
    assert B <= SMH_GEMV_MAX_M and p.n_total == (H + 2 * Hkv) * D and p.buf.dtype == torch.float32
    _need_gpu(p.buf, cache_k, cache_v, cache_ks, cache_vs, t_dev, pos_dev)
    if prefix_k is not None:
        assert prefix_k.is_contiguous() and prefix_v.is_contiguous() and prefix_k.dtype == torch.float16 and P <= prefix_k.shape[-3]
    else:
        assert P == 0
    assert cache_k.dtype == torch.int8 and cache_ks.dtype == torch.float16 and t_dev.dtype == torch.int32
    out = torch.empty((B, H, D), dtype=torch.float16, device=p.buf.device)
    ws = attn_qkv_workspace(p.buf.device, B, H, P) if single_launch else attn_workspace(p.buf.device, B, H, P)
    check(lib.smh_shared_prefix_attn_qkv(p.buf.data_ptr(), p.ksplit, out.data_ptr(), B, H, Hkv, D, cos.data_ptr(), sin.data_ptr(),
                                         pos_dev.data_ptr(), _ptr(prefix_k), _ptr(prefix_v), int(P),
                                         cache_k.data_ptr(), cache_ks.data_ptr(), cache_v.data_ptr(), cache_vs.data_ptr(), int(Smax),
                                         t_dev.data_ptr(), _ptr(pages), pages.stride(0) if pages is not None else 0,
                                         int(bool(single_launch)), ws.data_ptr(), ws.numel(), _stream()),
          "smh_shared_prefix_attn_qkv")
    return out


def prefill_attn(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """Causal attention over one prompt: q [S,H,128], k/v [S,Hkv,128] -> [S,H,128]."""
    lib = _lib.load()
    _need_gpu(q, k, v)
    assert q.is_contiguous() and k.is_contiguous() and v.is_contiguous()
    assert q.dtype == torch.float16 and k.dtype == torch.float16 and v.dtype == torch.float16
    S, H, D = q.shape
    out = torch.empty_like(q)
    check(lib.smh_prefill_attn(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), S, H, k.shape[1], D,
                               _stream()), "smh_prefill_attn")
    return out




def flash_attn(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, B: int, L: int, H: int, D: int) -> torch.Tensor:
    """Drop-in for triton_kernels.flash_attn (triton_kernels.py:621-647): one query per (branch, head) against
    that branch's own L keys.  q [B,H,D], k/v [B,H,L,D] fp16 -> [B,H,D] fp16.  The keys are brought into the
    token-major layout of the decode attention kernel ([B,L,H,D], one copy) and run as a suffix without prefix;
    scores and the softmax state are fp32 (the reference keeps them in fp16)."""
    _need_gpu(q, k, v)
    assert q.shape == (B, H, D) and k.shape == (B, H, L, D) and v.shape == (B, H, L, D)
    kt = k.transpose(1, 2).contiguous()
    vt = v.transpose(1, 2).contiguous()
    lens = torch.full((B,), L, dtype=torch.int32, device=q.device)
    return shared_prefix_attn(q.contiguous(), None, None, 0, suffix_k=kt, suffix_v=vt, Smax=L, lens=lens, lens_stride=1,
                              n_kv_heads=H)


def paged_prefix_attn(q: torch.Tensor, pages: torch.Tensor, lens: torch.Tensor, pool_k: torch.Tensor, pool_v: torch.Tensor,
                      pool_ks: Optional[torch.Tensor] = None, pool_vs: Optional[torch.Tensor] = None, head_major: bool = False,
                      prefix_k: Optional[torch.Tensor] = None, prefix_v: Optional[torch.Tensor] = None, P: int = 0,
                      prefix_head_major: bool = False, cur_k: Optional[torch.Tensor] = None, cur_v: Optional[torch.Tensor] = None,
                      lens_stride: int = 1, single_launch: bool = False) -> torch.Tensor:
    """Tree attention: out[b,h] = softmax(q[b,h] . K_b^T / sqrt(D)) . V_b with K_b = prefix[:P] (shared) || the pool rows
    pages[b, :lens[b]] || cur_k[b].  The rows are looked up inside the kernel (nothing is gathered or copied).
    pool: fp16 [rows, Hkv, D] (or [Hkv, rows, D] with head_major) or Q4_0 rows int8 [rows, Hkv, 64] + scales fp16
    [rows, Hkv, 2]; pages: int16 / int32 / int64 [B, L] (possibly a column slice of a wider table); lens int32 on the device,
    cut to L inside the kernel."""
    lib = _lib.load()
    _need_gpu(q, pages, lens, pool_k, pool_v)
    assert q.is_contiguous() and q.dtype == torch.float16 and q.dim() == 3
    B, H, D = q.shape
    assert pages.dim() == 2 and pages.shape[0] >= B and pages.stride(1) == 1 and pages.dtype in (torch.int16, torch.int32, torch.int64)
    assert lens.dtype == torch.int32
    assert pool_k.is_contiguous() and pool_v.is_contiguous() and pool_k.shape == pool_v.shape
    if pool_k.dtype == torch.float16:
        fmt = SMH_KV_FP16
        assert pool_k.dim() == 3 and pool_k.shape[2] == D
        Hkv = pool_k.shape[0] if head_major else pool_k.shape[1]
        rows = pool_k.shape[1] if head_major else pool_k.shape[0]
        row_stride, head_stride = (D, rows * D) if head_major else (0, 0)
    else:
        fmt = SMH_KV_Q40
        assert pool_k.dtype == torch.int8 and pool_ks is not None and pool_vs is not None and not head_major
        assert pool_ks.dtype == torch.float16 and pool_vs.dtype == torch.float16 and pool_ks.is_contiguous() and pool_vs.is_contiguous()
        assert pool_k.dim() == 3 and pool_k.shape[2] == 64
        Hkv = pool_k.shape[1]
        rows = pool_k.shape[0]
        row_stride = head_stride = 0
    assert H % Hkv == 0
    p_row = p_head = 0
    if prefix_k is not None and P > 0:
        assert prefix_k.is_contiguous() and prefix_v.is_contiguous() and prefix_k.dtype == torch.float16 and prefix_k.dim() == 3
        if prefix_head_major:
            assert prefix_k.shape[0] == Hkv and P <= prefix_k.shape[1]
            p_row, p_head = D, prefix_k.shape[1] * D
        else:
            assert prefix_k.shape[1] == Hkv and P <= prefix_k.shape[0]
    else:
        P = 0
    if cur_k is not None:
        assert cur_k.is_contiguous() and cur_v.is_contiguous() and cur_k.dtype == torch.float16 and cur_k.shape == (B, Hkv, D)
    out = torch.empty_like(q)
    one = bool(single_launch) and B * (H // Hkv) <= 128
    ws = attn_qkv_workspace(q.device, B, H, P) if one else attn_workspace(q.device, B, H, P)
    check(lib.smh_paged_prefix_attn(q.data_ptr(), out.data_ptr(), B, H, Hkv, D, _ptr(prefix_k) if P else None, _ptr(prefix_v) if P else None,
                                    int(P), p_row, p_head, fmt, pool_k.data_ptr(), pool_v.data_ptr(), _ptr(pool_ks), _ptr(pool_vs),
                                    row_stride, head_stride, int(rows), pages.data_ptr(), pages.element_size(), pages.stride(0), pages.shape[1],
                                    lens.data_ptr(), int(lens_stride), _ptr(cur_k), _ptr(cur_v), int(one), ws.data_ptr(), ws.numel(), _stream()),
          "smh_paged_prefix_attn")
    return out


def page_fork(table: torch.Tensor, origin: int, curr: int, forks: int, n: int) -> None:
    """table[curr : curr + forks, :n] = table[origin, :n] for an int32 page table [rows, stride]: the fork of a branch
    when its rows are shared through the table instead of copied."""
    lib = _lib.load()
    _need_gpu(table)
    assert table.dtype == torch.int32 and table.dim() == 2 and table.is_contiguous()
    check(lib.smh_page_fork(table.data_ptr(), table.shape[0], table.shape[1], int(origin), int(curr), int(forks), int(n), _stream()),
          "smh_page_fork")


def page_flash_attn(p: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, P: int, B: int, L: int, H: int,
                    D: int) -> torch.Tensor:
    """Drop-in for triton_kernels.page_flash_attn (triton_kernels.py:764-789): branch b attends to the L pages
    p[b, :] of the page pools k/v [H,P,D].  p [B,L] integer page ids, q [B,H,D] -> [B,H,D] fp16.  The pools are read
    where they lie, through the page table (no gather, no layout copy); scores and the softmax state are fp32 (the
    reference keeps them in fp16)."""
    _need_gpu(p, q, k, v)
    assert p.shape == (B, L) and q.shape == (B, H, D) and k.shape == (H, P, D) and v.shape == (H, P, D)
    lens = torch.full((1,), L, dtype=torch.int32, device=q.device)
    return paged_prefix_attn(q.contiguous(), p if p.stride(1) == 1 else p.contiguous(), lens, k.contiguous(), v.contiguous(),
                             head_major=True, lens_stride=0)


def chunk_attn(p: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, P: int, B: int, L: int, H: int,
               D: int, offset: int) -> torch.Tensor:
    """The intended result of triton_kernels.chunk_attn (triton_kernels.py:1150-1231): the first `offset` pages of
    the pools k/v [H,P,D] are one chunk that every branch attends to (no paging: pool rows 0..offset-1 in order),
    followed by the branch's own pages p[b, offset:L].  p [B,L] integer page ids, q [B,H,D] -> [B,H,D] fp16; equal
    to page_flash_attn whenever p[b, :offset] == arange(offset).  The reference's two kernels do not combine
    their softmax states correctly (base-2 against natural maxima, the first kernel's output not reloaded), so
    this follows the docstring of the reference function, not its output.  The shared chunk is the prefix of the
    decode attention kernel (staged once in LDS for all branches, read from the pool in place), the own pages are looked
    up through the page table inside the kernel."""
    _need_gpu(p, q, k, v)
    assert p.shape == (B, L) and q.shape == (B, H, D) and k.shape == (H, P, D) and v.shape == (H, P, D)
    assert 0 <= offset <= L and offset <= P
    k, v = k.contiguous(), v.contiguous()
    p = p if p.stride(1) == 1 else p.contiguous()
    lens = torch.full((1,), L - offset, dtype=torch.int32, device=q.device)
    own = p[:, offset:] if offset < L else p[:, :1]                    # a view: same table, first own page
    return paged_prefix_attn(q.contiguous(), own, lens, k, v, head_major=True, prefix_k=k, prefix_v=v, P=offset,
                             prefix_head_major=True, lens_stride=0)
