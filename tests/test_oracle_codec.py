"""Pins for the oracle's Q4_0 codec (fp16_to_int4.py:52-96 of the reference): three independent
implementations (torch CPU, numpy float16, integer-only C) must agree bit for bit, and the
quantiser must satisfy the invariants the format implies."""
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import q40_oracle as O


def _bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def _same_or_both_nan(a: np.ndarray, b: np.ndarray) -> bool:
    fa, fb = a.view(np.float16), b.view(np.float16)
    return bool(np.all((a == b) | (np.isnan(fa) & np.isnan(fb))))


def test_dequant_exhaustive_three_ways(cref):
    """every nibble pattern x every fp16 scale bit pattern"""
    table_c = np.zeros(16 * 65536, dtype=np.uint16)
    cref.q40_ref_dequant_table(table_c.ctypes.data)
    table_c = table_c.reshape(16, 65536)
    table_np = O.np_dequant_table()
    assert _same_or_both_nan(table_c, table_np)
    # torch: pack pattern p in the high nibble and 15-p in the low nibble of each byte
    scales = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.float16)
    for p in range(16):
        byte = ((p << 4) | (15 - p)) & 0xFF
        byte = byte - 256 if byte >= 128 else byte
        w = torch.full((32768, 64), byte, dtype=torch.int8)       # 32768 rows -> 65536 groups
        deq = O.dequantize_q40(w, scales.view(-1, 1), 64, (65536, 64))
        got = _bits(deq)
        assert _same_or_both_nan(got[0::2, 0], table_c[p, 0::2])          # high nibble rows use even scales
        assert _same_or_both_nan(got[1::2, 0], table_c[15 - p, 1::2])     # low nibble rows use odd scales
        assert np.all(got == got[:, :1])


def test_nibble_sign_extension():
    """0x8 decodes to -8, 0xF to -1 ("DO NOT JUST MASK", fp16_to_int4.py:91)"""
    w = torch.tensor([[-128 + 0x0F] * 64], dtype=torch.int8)    # byte 0x8F
    s = torch.tensor([[1.0], [1.0]], dtype=torch.float16)
    d = O.dequantize_q40(w, s, 64, (2, 64))
    assert torch.all(d[0] == -8) and torch.all(d[1] == -1)


def test_scale_true_division_all_absmax(cref):
    """scale = fp16(absmax / 7) with a true division, for every finite fp16 absmax"""
    amax = torch.arange(0, 0x7C00, dtype=torch.int32).to(torch.int16).view(torch.float16)
    got = _bits((amax / 7.0).type(torch.float16))
    want = np.array([cref.q40_ref_scale(int(a)) for a in range(0x7C00)], dtype=np.uint16)
    assert np.array_equal(got, want)
    # numpy as third opinion (float32 divide, one rounding to half)
    want_np = (np.arange(0x7C00, dtype=np.uint16).view(np.float16).astype(np.float32) / np.float32(7.0)).astype(np.float16)
    assert np.array_equal(got, want_np.view(np.uint16))


def test_quantize_matches_c_and_layout(cref):
    g = torch.Generator().manual_seed(0)
    x = (torch.randn((512, 64), generator=g) * 0.02).to(torch.float16)
    x[3] = 0                                   # all-zero group: scale 0, NaN quotient, code 0
    x[5, 7] = 6.5e4                            # near fp16 max
    x[6] = x[6] * 1e-4                         # subnormal territory
    w, s = O.quantize_q40(x, 64)
    assert w.shape == (256, 64) and s.shape == (512, 1) and w.dtype == torch.int8 and s.dtype == torch.float16
    wc = np.zeros((256, 64), dtype=np.int8)
    sc = np.zeros(512, dtype=np.uint16)
    xin = _bits(x).copy()
    cref.q40_ref_quantize(xin.ctypes.data, 512, wc.ctypes.data, sc.ctypes.data)
    assert np.array_equal(sc, _bits(s).ravel())
    assert np.array_equal(wc, w.numpy())
    # C dequant of the torch-quantised data == torch dequant
    out = np.zeros(256 * 128, dtype=np.uint16)
    cref.q40_ref_dequantize(w.numpy().ctypes.data, _bits(s).ctypes.data, 256, out.ctypes.data)
    assert _same_or_both_nan(out, _bits(O.dequantize_q40(w, s, 64, (512, 64))).ravel())


def test_quantizer_invariants():
    g = torch.Generator().manual_seed(1)
    x = (torch.randn((1024, 64), generator=g) * 0.5).to(torch.float16)
    w, s = O.quantize_q40(x, 64)
    codes = O.unpack_codes(w)
    assert int(codes.min()) >= -7 and int(codes.max()) <= 7
    assert torch.all(codes.abs().max(dim=1).values == 7)          # the absmax element maps to +-7
    deq = O.dequantize_q40(w, s, 64, x.shape)
    err = (deq.double() - x.double()).abs()
    sd = s.double()
    # half a step plus the fp16 roundings of the quotient and of the product
    assert torch.all(err <= sd * 0.5 + 8 * sd * 2.0 ** -10 + 1e-12)
    # idempotence: re-quantising the dequantised values reproduces codes and scales
    w2, s2 = O.quantize_q40(deq, 64)
    assert torch.equal(s2, s) and torch.equal(w2, w)


def test_quantize_tiny_groups_exact_rationals():
    """brute force: codes equal round-half-even of the exactly computed fp16 quotient"""
    g = torch.Generator().manual_seed(2)
    x = (torch.randn((2, 64), generator=g)).to(torch.float16)
    x[0, :8] = torch.tensor([0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 3.5, 7.0], dtype=torch.float16)
    x[0, 8:] = 0
    w, s = O.quantize_q40(x, 64)
    codes = O.unpack_codes(w)
    for r in range(2):
        sc = Fraction(float(s[r, 0]))
        assert sc == Fraction(float(np.float16(np.float32(float(x[r].abs().max())) / np.float32(7.0))))
        for j in range(64):
            quo = float(np.float16(np.float32(float(x[r, j])) / np.float32(float(s[r, 0]))))
            fl = Fraction(quo)
            lo = fl.numerator // fl.denominator
            frac = fl - lo
            want = lo if frac < Fraction(1, 2) else lo + 1 if frac > Fraction(1, 2) else (lo if lo % 2 == 0 else lo + 1)
            assert int(codes[r, j]) == want
    # the hand-made ties in row 0 (scale exactly 1): .5 -> 0, 1.5 -> 2, 2.5 -> 2, 3.5 -> 4
    assert codes[0, :8].tolist() == [0, 0, 2, -2, 2, -2, 4, 7]


def test_weight_layout_byte_map():
    """W^T[k,n] lives in byte k*(N/2) + (n//128)*64 + n%64, high nibble iff n%128 < 64; scale s[k, n//64]"""
    K, N = 8, 256
    g = torch.Generator().manual_seed(3)
    v = (torch.randn((N, K), generator=g) * 0.02).to(torch.float16)
    w, s, shp = O.quantize_weight(v)
    assert tuple(shp) == (N, K) and w.shape == (K * N // 128, 64) and s.shape == (K * N // 64, 1)
    deq = O.dequantize_q40(w, s, 64, (K, N))
    wb = w.view(-1).numpy().view(np.uint8)
    sf = s.view(-1)
    for k in range(K):
        for n in range(N):
            byte, high, sidx = O.weight_byte_index(k, n, N)
            nib = (wb[byte] >> 4) if high else (wb[byte] & 15)
            q = int(nib) - 16 if nib >= 8 else int(nib)
            want = torch.tensor(q, dtype=torch.float16) * sf[sidx]
            assert _bits(want.reshape(1))[0] == _bits(deq[k, n].reshape(1))[0]
    # and the dequantised matrix approximates v^T
    assert (deq.float() - v.t().float()).abs().max() <= s.float().max() * 0.51


# ---- the block-of-32 flavour that the benchmark's first configuration spells out ----------------------------------
def test_block32_dequant_every_nibble_and_scale():
    """(q - 8) * scale for all 16 nibbles x all 65536 fp16 scale patterns, against numpy float16 (an independent fp16
    multiply) - and against exact integer arithmetic where the product needs no rounding."""
    scales = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.float16)          # every bit pattern
    for q in range(16):
        byte = torch.full((65536, 16), q | (q << 4), dtype=torch.uint8)
        got = O.dequantize_gq40(byte, scales, (65536, 32))
        with np.errstate(over="ignore", invalid="ignore"):
            want = (np.float16(q - 8) * scales.numpy().astype(np.float16)).astype(np.float16)
        g = got[:, 0].numpy()
        same = (g.view(np.uint16) == want.view(np.uint16)) | (np.isnan(g) & np.isnan(want))
        assert same.all(), q
        assert torch.equal(got[:, 0].view(torch.int16), got[:, 31].view(torch.int16))              # both nibbles, every position
    # powers of two: the product is exact, so it must equal plain integer scaling
    s2 = torch.tensor([2.0 ** e for e in range(-10, 6)], dtype=torch.float16)
    by = torch.arange(16, dtype=torch.uint8).repeat(16, 1)                                        # low nibble j, high nibble 0
    d = O.dequantize_gq40(by.contiguous(), s2, (16, 32))
    for i in range(16):
        assert d[i, :16].tolist() == [(j - 8) * float(s2[i]) for j in range(16)]
        assert d[i, 16:].tolist() == [-8 * float(s2[i])] * 16


def test_block32_quantiser_invariants_and_layout():
    g = torch.Generator().manual_seed(5)
    w = (torch.randn((64, 128), generator=g) * 0.02).half()
    w[3] = 0                                                                                      # an all-zero block row: 0 / 0
    packed, scale = O.quantize_gq40(w)
    assert packed.shape == (64 * 4, 16) and packed.dtype == torch.uint8 and scale.shape == (256,)
    blocks = w.reshape(-1, 32)
    assert torch.equal(scale, (blocks.abs().max(1).values.float() / 8.0).half())                   # true division, one rounding
    deq = O.dequantize_gq40(packed, scale, w.shape)
    err = (deq.float() - w.float()).abs().reshape(-1, 32)
    sc = scale.float()[:, None]
    at_top = blocks.float() >= 7.5 * sc                                                           # would round to 16: cut to 15
    slack = blocks.float().abs() * 2.0 ** -10 + 1e-7                    # the fp16 roundings of the quotient and of the product
    assert bool((err[~at_top] <= (sc.expand_as(err) * 0.5 + slack)[~at_top]).all())
    assert bool((err[at_top] <= (sc.expand_as(err) * 1.0 + slack)[at_top]).all()) and int(at_top.sum()) > 0
    assert bool((deq[3] == 0).all()) and bool((packed[12:16] == 0x88).all())                       # 0 / 0 -> q = 8 -> value 0
    # element j in the low nibble of byte j, element j + 16 in the high nibble
    q = torch.round(blocks / scale[:, None]).float().nan_to_num(0.0, posinf=8.0, neginf=-8.0).to(torch.int32).add(8).clamp(0, 15)
    assert torch.equal(packed.to(torch.int32) & 15, q[:, :16]) and torch.equal(packed.to(torch.int32) >> 4, q[:, 16:])
    # the negative end is exact: -absmax -> q = 0 -> value -8 * scale
    lo = blocks.float().min(1).values
    neg = lo <= -blocks.abs().max(1).values.float()
    assert bool(((packed.to(torch.int32) & 15).min(1).values.minimum((packed.to(torch.int32) >> 4).min(1).values)[neg & (scale > 0)] == 0).all())
    # re-quantising what was dequantised reproduces codes and scales where the block's extreme code is -8 (scale recoverable)
    p2, s2 = O.quantize_gq40(deq)
    keep = neg & (scale > 0)
    assert torch.equal(p2[keep], packed[keep]) and torch.equal(s2[keep], scale[keep])
