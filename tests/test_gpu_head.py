"""The fp16 vocabulary projection (lm_head) and the embedding gather against their closed forms: a dense product in
double precision rounded once to fp16 (what nn.Linear without bias computes at hf_model_q40_kv_shared.py:509, within
the tolerance BASELINE.json states for matmul outputs: 1e-2 relative / 2e-3 absolute) and plain row indexing."""
import pytest
import torch

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-2, 2e-3


def _ref(x, w):
    return (x.double() @ w.double().t())


def _check(M, N, K, seed):
    from spec_mcts_amd import kernels as Kn
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((M, K), generator=g).half()
    w = (torch.randn((N, K), generator=g) * 0.02).half()
    got = Kn.f16_linear(x.cuda(), w.cuda()).cpu()
    assert got.shape == (M, N) and got.dtype == torch.float16
    want = _ref(x, w)
    err = (got.double() - want).abs()
    assert bool((err <= ATOL + RTOL * want.abs()).all()), f"M={M} N={N} K={K}: max err {float(err.max())}"
    # tighter: fp32 accumulation and one rounding stay within one fp16 ulp of the exact value
    assert float((err / want.abs().clamp_min(0.25)).max()) < 2e-3
    return x, w, got


@pytest.mark.parametrize("M", [1, 10, 100])
def test_lm_head_at_vocab_32016(M):
    _check(M, 32016, 4096, 500 + M)


@pytest.mark.parametrize("M,N,K", [(1, 1, 64), (3, 320, 256), (16, 127, 128), (17, 129, 192), (130, 384, 512), (257, 200, 64), (5, 8192, 8192)])
def test_lm_head_ragged_shapes(M, N, K):
    _check(M, N, K, 600 + M + N)


def test_lm_head_one_hot_rows_return_weight_columns_exactly():
    from spec_mcts_amd import kernels as Kn
    N, K = 1000, 256
    g = torch.Generator().manual_seed(700)
    w = (torch.randn((N, K), generator=g) * 0.02).half()
    ks = [0, 7, 63, 64, 129, 255]
    x = torch.zeros((len(ks), K), dtype=torch.float16)
    for i, k in enumerate(ks):
        x[i, k] = 1.0
    got = Kn.f16_linear(x.cuda(), w.cuda()).cpu()
    for i, k in enumerate(ks):
        assert torch.equal(got[i].view(torch.int16), w[:, k].contiguous().view(torch.int16))
    assert torch.equal(Kn.f16_linear(torch.zeros((2, K), dtype=torch.float16).cuda(), w.cuda()).cpu(), torch.zeros((2, N), dtype=torch.float16))


def test_lm_head_batched_input_and_out_argument():
    from spec_mcts_amd import kernels as Kn
    g = torch.Generator().manual_seed(701)
    x = torch.randn((3, 5, 128), generator=g).half().cuda()
    w = (torch.randn((77, 128), generator=g) * 0.1).half().cuda()
    out = torch.empty((3, 5, 77), dtype=torch.float16, device="cuda:0")
    got = Kn.f16_linear(x, w, out=out)
    assert got.data_ptr() == out.data_ptr() and got.shape == (3, 5, 77)
    assert torch.equal(got.view(15, 77), Kn.f16_linear(x.view(15, 128), w))


def test_embedding_gather():
    from spec_mcts_amd import kernels as Kn
    g = torch.Generator().manual_seed(702)
    table = torch.randn((32016, 4096), generator=g).half()
    tok = torch.randint(0, 32016, (7, 13), generator=g)
    tok[0, 0], tok[0, 1] = 0, 32015
    got = Kn.embedding(tok.cuda(), table.cuda()).cpu()
    assert got.shape == (7, 13, 4096)
    assert torch.equal(got.view(torch.int16), table[tok].view(torch.int16))
