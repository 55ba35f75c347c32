"""The persistent decode-step kernel (smh_decode_step) against the operator-by-operator path of the
same model and against the oracle: same arithmetic and rounding points, only fp32 summation order
differs (the K range of a matrix is cut differently)."""
import pytest
import torch

from oracle import q40_oracle as O

pytestmark = pytest.mark.gpu

MHA_SMALL = dict(dim=256, n_layers=2, n_heads=2, vocab_size=320, multiple_of=128, max_batch_size=16, max_seq_len=24,
                 max_prompt_seq_len=32)
# wide enough that matrix phases have more 32-row steps than workgroups (ranges cross unit borders,
# units have several contributors) and the prefix spans several 64-row attention chunks
MHA_WIDE = dict(dim=1024, n_layers=2, n_heads=8, vocab_size=512, multiple_of=256, max_batch_size=16, max_seq_len=16,
                max_prompt_seq_len=160)


def _build(cfg, seed, std=0.05):
    from spec_mcts_amd import ModelArgs
    from spec_mcts_amd.load_q40 import load_q40
    oargs = O.OracleArgs(**cfg)
    sd = O.random_q40_state_dict(oargs, seed=seed, std=std)
    model = load_q40(dict(sd), ModelArgs(**cfg), device="cuda:0")
    model.persistent = True
    model.persistent_max_branches = 16      # exercise the kernel over its whole range
    return oargs, sd, model


def _caches(model):
    return [t for l in model.layers for t in (l.attention.cache_k, l.attention.cache_k_s, l.attention.cache_v, l.attention.cache_v_s)]


@pytest.mark.parametrize("cfg,B,P", [(MHA_SMALL, 1, 7), (MHA_SMALL, 3, 19), (MHA_SMALL, 10, 32), (MHA_SMALL, 16, 5),
                                     (MHA_WIDE, 1, 150), (MHA_WIDE, 10, 70), (MHA_WIDE, 16, 129)])
def test_persistent_step_matches_operator_path(cfg, B, P):
    """Every step runs twice from the SAME cache state, operator by operator and as the persistent kernel.
    (Run back to back instead, the two paths drift apart: a Q4_0 code of the appended K/V row that sits on
    a rounding edge flips, and a flipped code moves that cache entry by a whole quantisation step.)"""
    print(f"case dim={cfg['dim']} B={B} P={P}", flush=True)
    _, _, model = _build(cfg, seed=60 + B)
    assert model._step_kernel(B, torch.device("cuda:0")) is not None, "the shape must be inside the persistent kernel"
    g = torch.Generator().manual_seed(B * 100 + P)
    prompt = torch.randint(0, cfg["vocab_size"], (1, P), generator=g)
    model.resetSeq()
    model(prompt.cuda(), 0)
    for s in range(6):
        tok = torch.randint(0, cfg["vocab_size"], (B, 1), generator=g).cuda()      # branches diverge
        before = [t.clone() for t in _caches(model)]
        model.persistent = False
        want = model(tok, P + s)[:, -1].float().cpu()
        after_want = [t.clone() for t in _caches(model)]
        for t, b in zip(_caches(model), before):
            t.copy_(b)
        model.persistent = True
        got = model(tok, P + s)[:, -1].float().cpu()
        torch.cuda.synchronize()
        model.check_step_kernels()
        assert torch.isfinite(got).all()
        assert torch.allclose(got, want, rtol=1e-2, atol=1e-2), f"step {s}: max diff {(got - want).abs().max()}"
        for t, w in zip(_caches(model), after_want):
            if t.dtype == torch.int8:
                assert (t != w).float().mean() < 0.01, f"step {s}: appended Q4_0 rows differ"
            else:
                assert torch.allclose(t.float(), w.float(), rtol=2e-2, atol=1e-4)
            t.copy_(w)


@pytest.mark.parametrize("B", [1, 10])
def test_persistent_tokens_match_oracle(B):
    from tests.test_gpu_model import _assert_tokens_match, _greedy_gpu
    cfg = dict(MHA_SMALL)
    oargs, sd, model = _build(cfg, seed=40)
    oracle = O.OracleTransformer(oargs, sd, dense=True)
    prompt = torch.randint(0, cfg["vocab_size"], (1, 17), generator=torch.Generator().manual_seed(140))
    want, margins = oracle.greedy(prompt, B, 12)
    model.persistent = True
    got = _greedy_gpu(model, prompt, B, 12)
    torch.cuda.synchronize()
    model.check_step_kernels()
    print("oracle top-1/top-2 margins:", ["%.3f" % m for m in margins])
    _assert_tokens_match(got, want, margins, min_steps=8)


def test_persistent_step_in_a_graph_replays():
    """GraphDecoder records the persistent step once and replays it; tokens equal the eager loop's"""
    from spec_mcts_amd.decode import GraphDecoder
    _, _, model = _build(MHA_SMALL, seed=61)
    prompt = torch.randint(0, MHA_SMALL["vocab_size"], (1, 11), generator=torch.Generator().manual_seed(161))
    outs = {}
    for use_graph in (False, True):
        dec = GraphDecoder(model, 4, use_graph=use_graph)
        dec.prefill(prompt)
        dec.capture()
        outs[use_graph] = dec.decode(9).cpu()
        torch.cuda.synchronize()
        model.check_step_kernels()
    assert torch.equal(outs[False], outs[True])


def test_shapes_outside_the_kernel_fall_back():
    from spec_mcts_amd import kernels as K
    assert not K.DecodeStepKernel.supports(17, 4096, 32, 32, 11008)       # too many branches
    assert not K.DecodeStepKernel.supports(4, 512, 4, 2, 1536)            # grouped-query attention
    assert K.DecodeStepKernel.supports(10, 4096, 32, 32, 11008)
