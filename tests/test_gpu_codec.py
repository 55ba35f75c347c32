"""GPU parity of the Q4_0 codec kernels against the oracle (bit-exact), through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import q40_oracle as O

pytestmark = pytest.mark.gpu


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _same_or_both_nan(a, b):
    fa, fb = a.view(np.float16), b.view(np.float16)
    return bool(np.all((a == b) | (np.isnan(fa) & np.isnan(fb))))


def test_dequant_exhaustive_bit_exact(cref):
    """every nibble pattern x every fp16 scale pattern, against the integer-only C table"""
    from spec_mcts_amd import kernels as K
    table = np.zeros(16 * 65536, dtype=np.uint16)
    cref.q40_ref_dequant_table(table.ctypes.data)
    table = table.reshape(16, 65536)
    # every row holds all 16 patterns in both nibble positions; row r uses scales (2r, 2r+1).
    # Two passes (the second with neighbouring scales swapped) cover all 16 x 65536 pairs for
    # both nibble positions.
    rows = 32768
    j = torch.arange(64)
    byte_row = ((j % 16) << 4) | ((j % 16 + j // 16) % 16)
    byte = byte_row[None, :].expand(rows, 64).contiguous()
    w = byte.to(torch.uint8).view(torch.int8)
    b = byte.numpy()
    r = np.arange(rows)[:, None]
    for swap in (0, 1):
        idx = torch.arange(65536, dtype=torch.int32) ^ swap
        scales = idx.to(torch.int16).view(torch.float16).view(-1, 1)
        got = _bits(K.deq_int40(w.cuda(), scales.cuda(), 64, (rows * 2, 64))).reshape(rows, 2, 64)
        assert _same_or_both_nan(got[:, 0, :], table[b >> 4, (2 * r) ^ swap])
        assert _same_or_both_nan(got[:, 1, :], table[b & 15, (2 * r + 1) ^ swap])


@pytest.mark.parametrize("shape", [(11008, 4096), (128, 64), (2, 64)])
def test_dequant_random_weights_bit_exact(shape):
    from spec_mcts_amd import kernels as K
    g = torch.Generator().manual_seed(0)
    v = (torch.randn(shape, generator=g) * 0.02).to(torch.float16)
    w, s = O.quantize_q40(v, 64)
    want = O.dequantize_q40(w, s, 64, shape)
    got = K.deq_int40(w.cuda(), s.cuda(), 64, shape)
    assert got.shape == tuple(shape) and got.dtype == torch.float16
    assert np.array_equal(_bits(got), _bits(want))


def test_quantize_matches_torch_rounding():
    from spec_mcts_amd import kernels as K
    g = torch.Generator().manual_seed(1)
    x = (torch.randn((4096, 64), generator=g) * 0.5).to(torch.float16)
    x[3] = 0                                            # 0/0 -> code 0, scale 0
    x[5, 7] = 6.0e4
    x[6] = x[6] * 1e-4                                   # subnormal scales
    x[8, :8] = torch.tensor([0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 3.5, 7.0], dtype=torch.float16)
    x[8, 8:] = 0                                         # exact ties: round half to even
    w_want, s_want = O.quantize_q40(x, 64)
    w_got, s_got = K.q_int40(x.cuda(), 64)
    assert w_got.shape == w_want.shape and s_got.shape == s_want.shape
    assert np.array_equal(_bits(s_got), _bits(s_want))
    assert torch.equal(w_got.cpu(), w_want)
    # round trip on the device reproduces the oracle's dequantised values
    back = K.deq_int40(w_got, s_got, 64, x.shape)
    assert np.array_equal(_bits(back), _bits(O.dequantize_q40(w_want, s_want, 64, x.shape)))
    # idempotence at full size: quantising dequantised data is the identity on (codes, scales)
    w2, s2 = K.q_int40(back, 64)
    assert torch.equal(w2, w_got) and torch.equal(s2, s_got)


def test_quantize_dispatch_host_tensor():
    from spec_mcts_amd import kernels as K
    g = torch.Generator().manual_seed(2)
    x = torch.randn((8, 64), generator=g).to(torch.bfloat16)
    w, s = K.quantize_q40(x, 64)
    w2, s2 = O.quantize_q40(x, 64)
    assert torch.equal(w, w2) and torch.equal(s, s2)
