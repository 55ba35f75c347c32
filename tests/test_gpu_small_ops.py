"""GPU parity of the small fused kernels (RMSNorm, SiLU*up, argmax, RoPE + Q4_0 KV append, fork)."""
import numpy as np
import pytest
import torch

from oracle import q40_oracle as O

pytestmark = pytest.mark.gpu


def _g(seed):
    return torch.Generator().manual_seed(seed)


@pytest.mark.parametrize("rows,dim", [(1, 4096), (10, 4096), (100, 4096), (3, 8192), (2, 256)])
def test_rmsnorm(rows, dim):
    from spec_mcts_amd import kernels as K
    x = torch.randn((rows, dim), generator=_g(1)).to(torch.float16)
    wt = (1 + 0.1 * torch.randn(dim, generator=_g(2))).to(torch.float16)
    got = K.rmsnorm(x.cuda(), wt.cuda(), 1e-5).cpu()
    want = O.rmsnorm(x, wt, 1e-5)
    # same cast points; the only freedom is the order of the fp32 sum of squares (<= 1 fp16 ulp)
    assert torch.allclose(got.float(), want.float(), rtol=2e-3, atol=1e-4)
    assert (got != want).float().mean() < 0.01


def test_silu_mul():
    from spec_mcts_amd import kernels as K
    a = (torch.randn(100 * 11008 + 3, generator=_g(3)) * 2).to(torch.float16)
    b = torch.randn(100 * 11008 + 3, generator=_g(4)).to(torch.float16)
    got = K.silu_mul(a.cuda(), b.cuda()).cpu()
    want = O.silu_mul(a, b)
    assert torch.allclose(got.float(), want.float(), rtol=2e-3, atol=1e-4)
    assert (got != want).float().mean() < 0.01


def test_argmax_lowest_index_on_ties():
    from spec_mcts_amd import kernels as K
    logits = torch.randn((100, 32016), generator=_g(5)).to(torch.float16)
    logits[0, 31000] = 9.0; logits[0, 17] = 9.0; logits[0, 5000] = 9.0     # three-way tie -> 17
    logits[1, 32015] = 50.0                                                  # last column
    logits[2] = 0.25                                                         # all equal -> 0
    got = K.argmax(logits.cuda()).cpu()
    assert got.dtype == torch.int64
    assert torch.equal(got, logits.float().argmax(-1))
    assert got[0] == 17 and got[1] == 32015 and got[2] == 0
    # strided rows (a [B,1,V] slice of a bigger buffer)
    big = torch.randn((4, 40000), generator=_g(6)).to(torch.float16).cuda()
    assert torch.equal(K.argmax(big[:, :32016]).cpu(), big[:, :32016].float().argmax(-1).cpu())


def test_rope_prefill_bit_exact():
    from spec_mcts_amd import kernels as K
    S, H, Hkv, D = 37, 8, 2, 128
    fc = O.precompute_freqs_cis(D, 64, 1e6)
    q = torch.randn((1, S, H, D), generator=_g(7)).to(torch.float16)
    k = torch.randn((1, S, Hkv, D), generator=_g(8)).to(torch.float16)
    qe, ke = O.apply_rotary_emb(q, k, fc[3:3 + S])
    cos, sin = fc.real.to(torch.float16).contiguous().cuda(), fc.imag.to(torch.float16).contiguous().cuda()
    qd, kd = q[0].clone().cuda(), k[0].clone().cuda()
    K.rope(qd, kd, cos, sin, 3)
    assert torch.equal(qd.cpu().view(torch.int16), qe[0].view(torch.int16))
    assert torch.equal(kd.cpu().view(torch.int16), ke[0].view(torch.int16))


def test_rope_append_kv_bit_exact():
    """decode step: rotate q,k at position pos; store Q4_0(k_rot), Q4_0(v) in row t of each branch"""
    from spec_mcts_amd import kernels as K
    B, H, Hkv, D, Smax, Bmax = 5, 8, 2, 128, 6, 7
    pos, t = 21, 4
    fc = O.precompute_freqs_cis(D, 64, 1e6)
    q = torch.randn((B, 1, H, D), generator=_g(9)).to(torch.float16)
    k = torch.randn((B, 1, Hkv, D), generator=_g(10)).to(torch.float16)
    v = torch.randn((B, 1, Hkv, D), generator=_g(11)).to(torch.float16)
    v[0, 0, 0, :64] = 0                                           # an all-zero group
    qe, ke = O.apply_rotary_emb(q, k, fc[pos:pos + 1])
    cos, sin = fc.real.to(torch.float16).contiguous().cuda(), fc.imag.to(torch.float16).contiguous().cuda()
    rows = Bmax * Smax * Hkv
    ck = torch.zeros((rows, 64), dtype=torch.int8).cuda(); cks = torch.zeros((rows * 2, 1), dtype=torch.float16).cuda()
    cv = torch.zeros((rows, 64), dtype=torch.int8).cuda(); cvs = torch.zeros((rows * 2, 1), dtype=torch.float16).cuda()
    qd, kd, vd = q[:, 0].clone().cuda(), k[:, 0].clone().cuda(), v[:, 0].clone().cuda()
    state = torch.tensor([pos, t], dtype=torch.int32).cuda()
    K.rope_append_kv(qd, kd, vd, cos, sin, state[0:1], ck, cks, cv, cvs, Smax, state[1:2])
    assert torch.equal(qd.cpu().view(torch.int16), qe[:, 0].view(torch.int16))
    assert torch.equal(kd.cpu().view(torch.int16), ke[:, 0].view(torch.int16))
    wk, sk = O.quantize_q40(ke[:, 0], 64)                          # [B*Hkv, 64], [B*Hkv*2, 1]
    wv, sv = O.quantize_q40(v[:, 0], 64)
    ck4 = ck.cpu().view(Bmax, Smax, Hkv, 64); cks4 = cks.cpu().view(Bmax, Smax, Hkv, 2)
    cv4 = cv.cpu().view(Bmax, Smax, Hkv, 64); cvs4 = cvs.cpu().view(Bmax, Smax, Hkv, 2)
    assert torch.equal(ck4[:B, t], wk.view(B, Hkv, 64)) and torch.equal(cv4[:B, t], wv.view(B, Hkv, 64))
    assert torch.equal(cks4[:B, t].view(torch.int16), sk.view(B, Hkv, 2).view(torch.int16))
    assert torch.equal(cvs4[:B, t].view(torch.int16), sv.view(B, Hkv, 2).view(torch.int16))
    # nothing else was touched
    ck4[:B, t] = 0; cv4[:B, t] = 0
    assert not ck4.any() and not cv4.any()


def test_kv_fork_copies_rows():
    from spec_mcts_amd import kernels as K
    Bmax, Smax, Hkv = 6, 4, 2
    rows = Bmax * Smax * Hkv
    c = torch.randint(-128, 127, (rows, 64), generator=_g(12), dtype=torch.int8)
    s = torch.randn((rows * 2, 1), generator=_g(13)).to(torch.float16)
    cd, sd_ = c.clone().cuda(), s.clone().cuda()
    K.kv_fork(cd, sd_, Bmax, 1, 3, 2)
    want_c = c.view(Bmax, -1).clone(); want_s = s.view(Bmax, -1).clone()
    want_c[3:5] = want_c[1]; want_s[3:5] = want_s[1]
    assert torch.equal(cd.cpu().view(Bmax, -1), want_c)
    assert torch.equal(sd_.cpu().view(Bmax, -1).view(torch.int16), want_s.view(torch.int16))


@pytest.mark.parametrize("rows,vocab,k,temperature", [(100, 32016, 32, 0.8), (3, 320, 5, 1.0), (7, 1000, 1, 1.3), (4, 50, 50, 2.0),
                                                      (5, 4096, 1000, 0.6), (2, 70000, 64, 1.0)])
def test_sample_topk_matches_the_oracle(rows, vocab, k, temperature):
    """same candidates, same fp16 probabilities, same draw for the same uniform numbers; where u * total falls within
    fp32 rounding of a boundary of the cumulative probabilities either neighbour is accepted"""
    from spec_mcts_amd import kernels as K
    g = torch.Generator().manual_seed(500 + vocab + k)
    logits = (torch.randn((rows, vocab), generator=g) * 2.5).half()
    p, idx = O.topk_probs(logits, temperature, k)
    cdf = p.float().cumsum(-1)
    for trial in range(4):
        u = torch.rand(rows, generator=g)
        want = O.sample_topk(logits, temperature, k, u)
        got = K.sample_topk(logits.cuda(), temperature, k, u.cuda()).cpu()
        for r in range(rows):
            if int(got[r]) == int(want[r]):
                continue
            pos = (idx[r] == int(got[r])).nonzero()
            assert len(pos) == 1, f"row {r}: token {int(got[r])} is not a candidate"
            j = int(pos[0])
            target = float(u[r]) * float(cdf[r, -1])
            edges = [float(cdf[r, j - 1]) if j else 0.0, float(cdf[r, j])]
            assert min(abs(e - target) for e in edges) < 1e-5, f"row {r}: drew candidate {j}, target {target}, interval {edges}"


def test_sample_topk_ties_take_the_lowest_indices_and_frequencies_follow_p():
    from spec_mcts_amd import kernels as K
    # ties: a row of few distinct values; the candidates must be those of the stable order
    logits = torch.tensor([[1.0, 3.0, 2.0, 3.0, 2.0, 2.0, 0.5, 3.0]], dtype=torch.float16).repeat(64, 1)
    p, idx = O.topk_probs(logits, 1.0, 5)                       # 3.0 at 1, 3, 7, then 2.0 at 2, 4 (not 5)
    assert idx[0].tolist() == [1, 3, 7, 2, 4]
    u = torch.linspace(0.0, 0.999, 64)
    got = K.sample_topk(logits.cuda(), 1.0, 5, u.cuda()).cpu()
    assert set(got.tolist()) <= {1, 3, 7, 2, 4} and 5 not in got.tolist()
    assert torch.equal(got, O.sample_topk(logits, 1.0, 5, u)) or (got != O.sample_topk(logits, 1.0, 5, u)).sum() <= 2
    # frequencies
    g = torch.Generator().manual_seed(9)
    row = (torch.randn((1, 2000), generator=g) * 2).half()
    n = 20000
    p, idx = O.topk_probs(row, 0.9, 8)
    draws = K.sample_topk(row.expand(n, -1).contiguous().cuda(), 0.9, 8, torch.rand(n, generator=g).cuda()).cpu()
    for j in range(8):
        freq = float((draws == idx[0, j]).float().mean()); pj = float(p[0, j])
        assert abs(freq - pj) < 4 * (pj * (1 - pj) / n) ** 0.5 + 1e-3


@pytest.mark.parametrize("rows,vocab,k,temperature,grid", [(100, 32016, 32, 0.8, 0), (6, 32016, 32, 1.0, 8), (3, 320, 5, 1.0, 2),
                                                           (7, 1000, 1, 1.3, 4), (4, 50, 50, 2.0, 2), (5, 4096, 1000, 0.6, 0)])
def test_sample_topk_filter_matches_the_oracle(rows, vocab, k, temperature, grid):
    """smh_sample_topk_filter (hf_model_q40.py:521-533) against the oracle: the same surviving tokens - every value equal to
    the k-th largest included, which a coarse grid of logits makes common - the same float32 probabilities and the same
    draw for the same uniform numbers, either neighbour accepted where the target is within rounding of a boundary"""
    from spec_mcts_amd import kernels as K
    g = torch.Generator().manual_seed(900 + vocab + k)
    logits = torch.randn((rows, vocab), generator=g) * 2.5
    logits = (torch.round(logits * grid) / grid if grid else logits).half()
    p = O.topk_filter_probs(logits, temperature, k)
    order = torch.argsort(logits.float(), dim=-1, descending=True, stable=True)
    cdf = torch.gather(p, 1, order).cumsum(-1)
    n_alive = (p > 0).sum(-1)
    assert grid == 0 or int((n_alive > k).sum()) > 0 or k in (1, vocab)          # the grid cases do hold ties at the k-th value
    for trial in range(4):
        u = torch.rand(rows, generator=g)
        want = O.sample_topk_filter(logits, temperature, k, u)
        got = K.sample_topk_filter(logits.cuda(), temperature, k, u.cuda()).cpu()
        for r in range(rows):
            if int(got[r]) == int(want[r]):
                continue
            assert float(p[r, int(got[r])]) > 0, f"row {r}: token {int(got[r])} was filtered out"
            j = int((order[r] == int(got[r])).nonzero()[0])
            target = float(u[r]) * float(cdf[r, int(n_alive[r]) - 1])
            edges = [float(cdf[r, j - 1]) if j else 0.0, float(cdf[r, j])]
            assert min(abs(e - target) for e in edges) < 1e-5, f"row {r}: drew candidate {j}, target {target}, interval {edges}"
    # the last surviving tie is reachable: u just below 1 draws the highest index among the values equal to the k-th
    u = torch.full((rows,), 0.9999999)
    got = K.sample_topk_filter(logits.cuda(), temperature, k, u.cuda()).cpu()
    for r in range(rows):
        assert int(got[r]) == int(order[r, int(n_alive[r]) - 1])


def test_flat_cache_generate_samples_with_the_kernel():
    """hf_model_q40.Transformer.generate with a temperature and top_k draws through smh_sample_topk_filter: with torch's
    generator seeded the same way, the tokens equal those of the sampler called by hand on the same logits"""
    from spec_mcts_amd import hf_model_q40 as M, kernels as K
    from spec_mcts_amd.load_q40 import load_q40
    cfg = dict(dim=256, n_layers=1, n_heads=2, vocab_size=640, multiple_of=128, max_batch_size=3, max_seq_len=24)
    sd = O.random_q40_state_dict(O.OracleArgs(**cfg, max_prompt_seq_len=24), seed=38)
    model = load_q40(dict(sd), M.ModelArgs(**cfg), device="cuda:0", model_cls=M.Transformer)
    prompt = torch.randint(3, 640, (1, 5), generator=torch.Generator().manual_seed(39)).cuda()
    calls = []
    real = K.sample_topk_filter
    K.sample_topk_filter = lambda *a, **kw: (calls.append(1), real(*a, **kw))[1]
    try:
        torch.manual_seed(11)
        res, lens = model.generate(prompt, 3, 6, temperature=0.8, top_k=7)
    finally:
        K.sample_topk_filter = real
    assert len(calls) == 6 and res.shape == (3, 6) and int(res.max()) < 640
    model.fused_sampler = False
    torch.manual_seed(11)
    res2, _ = model.generate(prompt, 3, 6, temperature=0.8, top_k=7)              # torch's own sampler: another stream of draws
    assert res2.shape == (3, 6)


def test_detect_terminal_matches_the_oracle():
    """smh_detect_terminal against the oracle's detectTerminal on token streams with the terminal sequence, near
    matches and end-of-sequence tokens spliced in, 300 branches, 80 steps, state carried on the device: bit-exact"""
    from spec_mcts_amd import kernels as K
    seq = torch.tensor([29961, 29914, 20055, 4690, 1164, 29962], dtype=torch.int64)
    g = torch.Generator().manual_seed(91)
    B, T = 300, 80
    toks = torch.randint(0, 50, (B, T), generator=g)
    toks = torch.where(toks < 18, seq[toks % 6], toks + 100)          # a third of the tokens come from the sequence
    toks[toks == 131] = 2                                              # some end-of-sequence tokens
    for b in range(0, B, 3):
        at = int(torch.randint(0, T - 6, (1,), generator=g))
        toks[b, at:at + 6] = seq
    st_o = torch.zeros(B, dtype=torch.int32)
    st_d = st_o.cuda()
    seq_d, toks_d = seq.cuda(), toks.cuda()
    ends = 0
    for i in range(T):
        e_o, st_o = O.detect_terminal(toks[:, i].contiguous(), st_o, seq)
        e_d, st_d = K.detect_terminal(toks_d[:, i].contiguous(), st_d, seq_d)
        assert torch.equal(e_d.cpu(), e_o) and torch.equal(st_d.cpu(), st_o), f"step {i}"
        ends += int(e_o.sum())
    assert ends >= B // 3
    # no branches: nothing to do
    e, s_ = K.detect_terminal(toks_d[:0, 0].contiguous(), st_d[:0], seq_d)
    assert e.numel() == 0 and s_.numel() == 0
