"""The drop-in model where the decode step leaves the small-batch kernels: more than 16 branches (LDS/MFMA
GEMM, K-slice slabs, their consumers) and the layer shapes of the 70B architecture (BASELINE
configs[4]: dim 8192, 64 heads over 8 KV heads, FFN 28672), each against the oracle's dense restatement.

Branches are given DIFFERENT tokens, so a row mix-up between branches cannot cancel out, and several decode
steps are taken, so the later ones read suffix rows the earlier ones appended."""
import pytest
import torch

from oracle import q40_oracle as O
from tests.sync_state import sync_prefix, sync_suffix_row

pytestmark = pytest.mark.gpu


def _build(cfg, seed, std):
    from spec_mcts_amd import ModelArgs
    from spec_mcts_amd.load_q40 import load_q40
    oargs = O.OracleArgs(**cfg)
    sd = O.random_q40_state_dict(oargs, seed=seed, std=std)
    model = load_q40(dict(sd), ModelArgs(**cfg), device="cuda:0")
    return oargs, sd, model


def _steps(cfg, seed, B, P, std, rtol, atol, steps=3):
    oargs, sd, model = _build(cfg, seed, std)
    oracle = O.OracleTransformer(oargs, sd, dense=True)
    gen = torch.Generator().manual_seed(seed + 100)
    prompt = torch.randint(0, cfg["vocab_size"], (1, P), generator=gen)
    want0 = oracle.forward(prompt, 0)
    got0 = model(prompt.cuda(), 0).cpu()
    assert torch.allclose(got0.float(), want0.float(), rtol=rtol, atol=atol)
    # Every step starts from the oracle's cache state (tests/sync_state.py), so every step and every branch is held to
    # the tolerance: steps after the first read the suffix rows the earlier ones appended.
    sync_prefix(model, oracle)
    for step in range(steps):
        tok = torch.randint(0, cfg["vocab_size"], (B, 1), generator=gen)
        want = oracle.forward(tok, P + step)
        got = model(tok.cuda(), P + step).cpu()
        assert got.shape == want.shape and got.dtype == torch.float16
        diff = (got.float() - want.float()).abs().reshape(B, -1)
        bound = atol + rtol * want.float().abs().reshape(B, -1)
        row_ok = (diff <= bound).all(dim=1)
        print(f"B={B} step {step}: largest logit difference {float(diff.max()):.4f}, branches within tolerance {int(row_ok.sum())}/{B}")
        assert bool(row_ok.all()), f"step {step}: largest difference {float(diff.max())}, branches outside the tolerance {torch.nonzero(~row_ok).flatten().tolist()}"
        sync_suffix_row(model, oracle, B, step)


MANY = dict(dim=256, n_layers=2, n_heads=2, vocab_size=320, multiple_of=128, max_batch_size=40, max_seq_len=8,
            max_prompt_seq_len=32)
MANY_GQA = dict(dim=512, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=384, multiple_of=128, max_batch_size=112,
                max_seq_len=8, max_prompt_seq_len=48)


@pytest.mark.parametrize("cfg,seed,B", [(MANY, 70, 17), (MANY, 71, 40), (MANY_GQA, 72, 33), (MANY_GQA, 73, 100)])
def test_decode_logits_above_16_branches(cfg, seed, B):
    _steps(cfg, seed, B, P=21, std=0.05, rtol=1e-2, atol=1e-2)


ARCH_70B_LAYER = dict(dim=8192, n_layers=1, n_heads=64, n_kv_heads=8, vocab_size=512, multiple_of=4096,
                      ffn_dim_multiplier=1.3, max_batch_size=20, max_seq_len=8, max_prompt_seq_len=16)


@pytest.mark.parametrize("B,P", [(3, 9), (20, 9), (100, 2048)])
def test_70b_architecture_layer(B, P):
    """One layer with the 70B shapes (wq 8192x8192, wk/wv 1024x8192, w1/w3 28672x8192, w2 8192x28672, 8 query
    heads per KV head) through prefill and decode steps: GEMV at B=3, GEMM at B=20, and the workload of BASELINE
    configs[4] - 100 branches over a 2048-token shared prompt - at B=100."""
    cfg = dict(ARCH_70B_LAYER, max_batch_size=max(B, 20), max_prompt_seq_len=max(P, 16))
    assert O.ffn_hidden_dim(cfg["dim"], cfg["multiple_of"], cfg["ffn_dim_multiplier"]) == 28672
    _steps(cfg, 74, B, P=P, std=0.02, rtol=1e-2, atol=1e-2, steps=2 if P > 100 else 3)
