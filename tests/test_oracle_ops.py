"""Pins for the oracle's matmul, norm, RoPE, attention and whole-model composition: each is checked
against a library routine, a closed form in float64, or a special case with a known answer."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import q40_oracle as O


def _rand_q40(K, N, seed, std=0.02):
    g = torch.Generator().manual_seed(seed)
    v = (torch.randn((N, K), generator=g) * std).to(torch.float16)
    return O.quantize_weight(v)


def test_matmul_against_float64_and_one_hot():
    K, N = 256, 384
    w, s, _ = _rand_q40(K, N, 10)
    g = torch.Generator().manual_seed(11)
    a = torch.randn((5, K), generator=g).to(torch.float16)
    deq = O.dequantize_q40(w, s, 64, (K, N))
    want = (a.double() @ deq.double())
    got = O.matmul_q40(a, w, s, (K, N))
    assert torch.allclose(got.double(), want, rtol=1e-3, atol=1e-3)
    # one-hot rows pick single dequantised rows exactly; zero input gives zero
    eye = torch.zeros((3, K), dtype=torch.float16)
    eye[0, 0] = 1; eye[1, 63] = 1; eye[2, K - 1] = 1
    got = O.matmul_q40(eye, w, s, (K, N))
    assert torch.equal(got[0], deq[0]) and torch.equal(got[1], deq[63]) and torch.equal(got[2], deq[K - 1])
    assert torch.all(O.matmul_q40(torch.zeros((1, K), dtype=torch.float16), w, s, (K, N)) == 0)
    # the torch-only CPU path (dequant + F.linear) is the same function
    assert torch.equal(O.linear_q40_cpu_path(a, w, s, (N, K)), O.matmul_q40(a, w, s, (K, N)))


def test_rmsnorm_closed_form():
    g = torch.Generator().manual_seed(12)
    x = torch.randn((3, 512), generator=g).to(torch.float16)
    wt = (1 + 0.1 * torch.randn(512, generator=g)).to(torch.float16)
    got = O.rmsnorm(x, wt, 1e-5)
    xd = x.double()
    want = xd / torch.sqrt((xd ** 2).mean(-1, keepdim=True) + 1e-5) * wt.double()
    assert torch.allclose(got.double(), want, rtol=2e-3, atol=1e-4)
    # constant row: x/|x| = 1 -> output equals the weight (eps negligible)
    assert torch.equal(O.rmsnorm(torch.full((1, 512), 3.0, dtype=torch.float16), wt, 1e-12), wt[None])


def test_rope_table_and_rotation():
    D, T, theta = 128, 40, 1e6
    fc = O.precompute_freqs_cis(D, T, theta)
    assert fc.shape == (T, D // 2) and fc.dtype == torch.complex64
    t = np.arange(T)[:, None].astype(np.float64)
    inv = theta ** (-np.arange(0, D, 2).astype(np.float64) / D)
    assert np.allclose(fc.real.numpy(), np.cos(t * inv), atol=2e-6)
    assert np.allclose(fc.imag.numpy(), np.sin(t * inv), atol=2e-6)
    g = torch.Generator().manual_seed(13)
    q = torch.randn((2, T, 4, D), generator=g).to(torch.float16)
    k = torch.randn((2, T, 2, D), generator=g).to(torch.float16)
    qe, ke = O.apply_rotary_emb(q, k, fc)
    # position 0 is the identity
    assert torch.equal(qe[:, 0], q[:, 0]) and torch.equal(ke[:, 0], k[:, 0])
    # each (i, i+64) pair is rotated by angle t*inv_i: check against float64 and norm preservation
    qd = q.double()
    c = torch.from_numpy(np.cos(t * inv))[None, :, None, :]
    s_ = torch.from_numpy(np.sin(t * inv))[None, :, None, :]
    x1, x2 = qd[..., :64], qd[..., 64:]
    want = torch.cat((x1 * c - x2 * s_, x2 * c + x1 * s_), dim=-1)
    assert torch.allclose(qe.double(), want, atol=6e-3, rtol=0)
    n0 = (qd[..., :64] ** 2 + qd[..., 64:] ** 2)
    n1 = (qe.double()[..., :64] ** 2 + qe.double()[..., 64:] ** 2)
    assert torch.allclose(n0, n1, atol=3e-2, rtol=1e-2)


def test_silu_mul():
    g = torch.Generator().manual_seed(14)
    a = torch.randn(1000, generator=g).to(torch.float16)
    b = torch.randn(1000, generator=g).to(torch.float16)
    want = a.double() / (1 + torch.exp(-a.double())) * b.double()
    assert torch.allclose(O.silu_mul(a, b).double(), want, atol=2e-3, rtol=2e-3)
    assert torch.equal(O.silu_mul(a, b), F.silu(a) * b)          # same rounding points as torch's fp16 ops


def _attn_inputs(B, H, Hkv, D, P, S, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((B, H, D), generator=g).to(torch.float16)
    pk = torch.randn((P, Hkv, D), generator=g).to(torch.float16)
    pv = torch.randn((P, Hkv, D), generator=g).to(torch.float16)
    sk = torch.randn((B, S, Hkv, D), generator=g).to(torch.float16)
    sv = torch.randn((B, S, Hkv, D), generator=g).to(torch.float16)
    lens = torch.randint(0, S + 1, (B,), generator=g).tolist()
    return q, pk, pv, sk, sv, lens


@pytest.mark.parametrize("Hkv", [4, 2])
def test_attention_against_sdpa(Hkv):
    B, H, D, P, S = 5, 4, 128, 37, 9
    q, pk, pv, sk, sv, lens = _attn_inputs(B, H, Hkv, D, P, S, 20)
    lens[0] = 0; lens[1] = S
    got = O.shared_prefix_attention(q, pk, pv, sk, sv, lens)
    n_rep = H // Hkv
    for b in range(B):
        k = torch.cat((pk, sk[b, :lens[b]]), 0).repeat_interleave(n_rep, 1).transpose(0, 1).float()
        v = torch.cat((pv, sv[b, :lens[b]]), 0).repeat_interleave(n_rep, 1).transpose(0, 1).float()
        want = F.scaled_dot_product_attention(q[b].float()[:, None, :], k, v)[:, 0]
        assert torch.allclose(got[b].float(), want, atol=2e-3, rtol=1e-2)


def test_attention_special_cases_and_split_invariance():
    B, H, D, P, S = 3, 2, 128, 16, 8
    q, pk, pv, sk, sv, lens = _attn_inputs(B, H, H, D, P, S, 21)
    # all-equal scores (q = 0) -> mean of V over prefix + suffix
    z = torch.zeros_like(q)
    got = O.shared_prefix_attention(z, pk, pv, sk, sv, [S] * B)
    for b in range(B):
        want = torch.cat((pv, sv[b]), 0).float().mean(0)
        assert torch.allclose(got[b].float(), want, atol=2e-3)
    # one dominant key -> its V row
    pk2 = pk.clone(); pk2[5] = 0; pk2[5, :, 0] = 200.0
    q2 = torch.zeros_like(q); q2[..., 0] = 50.0
    got = O.shared_prefix_attention(q2, pk2 * 0 + pk2, pv, None, None, None)
    assert torch.allclose(got[0].float(), pv[5].float(), atol=1e-3)
    # moving tokens from the prefix into every branch's suffix changes nothing
    full = O.shared_prefix_attention(q, pk, pv, sk, sv, [S] * B)
    cut = 11
    sk2 = torch.cat((pk[cut:][None].expand(B, -1, -1, -1), sk), 1)
    sv2 = torch.cat((pv[cut:][None].expand(B, -1, -1, -1), sv), 1)
    moved = O.shared_prefix_attention(q, pk[:cut], pv[:cut], sk2, sv2, [S + P - cut] * B)
    assert torch.allclose(full.float(), moved.float(), atol=1e-3)


def test_causal_attention_against_sdpa():
    S, H, D = 19, 2, 128
    g = torch.Generator().manual_seed(22)
    q, k, v = (torch.randn((S, H, D), generator=g).to(torch.float16) for _ in range(3))
    got = O.causal_attention(q, k, v)
    want = F.scaled_dot_product_attention(q.transpose(0, 1).float(), k.transpose(0, 1).float(),
                                          v.transpose(0, 1).float(), is_causal=True).transpose(0, 1)
    assert torch.allclose(got.float(), want, atol=2e-3, rtol=1e-2)


TINY = dict(dim=256, n_layers=2, n_heads=2, vocab_size=320, multiple_of=128, max_batch_size=4,
            max_seq_len=8, max_prompt_seq_len=16)


def test_ffn_hidden_dim():
    assert O.ffn_hidden_dim(4096, 256, None) == 11008
    assert O.ffn_hidden_dim(8192, 4096, 1.3) == 28672


def test_model_dense_equals_q40_path_and_branches_agree():
    args = O.OracleArgs(**TINY)
    sd = O.random_q40_state_dict(args, seed=30, std=0.05)
    prompt = torch.randint(0, args.vocab_size, (1, 10), generator=torch.Generator().manual_seed(31))
    dense = O.OracleTransformer(args, sd, dense=True)
    q40 = O.OracleTransformer(args, sd, dense=False)
    t_dense, margins = dense.greedy(prompt, 3, 6)
    t_q40, _ = q40.greedy(prompt, 3, 6)
    assert torch.equal(t_dense, t_q40)
    assert torch.equal(t_dense[0], t_dense[1]) and torch.equal(t_dense[0], t_dense[2])
    assert len(margins) == 6 and all(m >= 0 for m in margins)


def test_model_incremental_equals_full_recompute_without_kv_quant():
    """prefill(P) + decode steps give the logits of prefill(P+t) at the same positions when the suffix
    KV is kept exact (the only approximation in the decode path is the Q4 KV round trip)."""
    args = O.OracleArgs(**TINY)
    sd = O.random_q40_state_dict(args, seed=32, std=0.05)
    g = torch.Generator().manual_seed(33)
    toks = torch.randint(0, args.vocab_size, (1, 13), generator=g)
    m = O.OracleTransformer(args, sd, dense=True, quantize_kv=False)
    full = m.forward(toks, 0)[0]                       # [13, vocab]
    m.reset()
    inc = [m.forward(toks[:, :10], 0)[0, -1]]
    for t in range(10, 13):
        inc.append(m.forward(toks[:, t:t + 1], t)[0, -1])
    inc = torch.stack(inc)
    assert torch.allclose(inc.float(), full[9:13].float(), atol=3e-2, rtol=3e-2)
    assert torch.equal(inc.argmax(-1), full[9:13].argmax(-1))


def test_per_branch_flavour_reduces_to_shared_flavour_without_kv_quantisation():
    """hf_model_q40's protocol (all positions in per-row caches) differs from the shared-prefix protocol only in
    that the PROMPT rows are seen through Q4_0 by later steps: with KV quantisation switched off both
    restatements must produce the same logits, prefill and decode, and with it on they must differ."""
    args = O.OracleArgs(dim=256, n_layers=2, n_heads=2, vocab_size=320, multiple_of=128, max_batch_size=3, max_seq_len=12,
                        max_prompt_seq_len=12)
    sd = O.random_q40_state_dict(args, seed=11, std=0.05)
    g = torch.Generator().manual_seed(12)
    prompt = torch.randint(0, 320, (1, 7), generator=g)
    toks = [torch.randint(0, 320, (3, 1), generator=g) for _ in range(3)]
    outs = {}
    for name, kw in (("shared", dict(quantize_kv=False)), ("rows", dict(quantize_kv=False, per_branch_kv=True)),
                     ("rows_q", dict(quantize_kv=True, per_branch_kv=True))):
        m = O.OracleTransformer(args, sd, dense=True, **kw)
        if name == "shared":
            res = [m.forward(prompt, 0)]
            m.fork(0, 1, 2)
        else:
            res = [m.forward(prompt.expand(3, -1), 0)[:1]]
        for s, t in enumerate(toks):
            res.append(m.forward(t, 7 + s))
        outs[name] = res
    for a, b in zip(outs["shared"], outs["rows"]):
        # same values up to the blocking of the host matmuls (one prompt row against three)
        assert torch.allclose(a.float(), b.float(), rtol=0, atol=4e-3)
    assert (outs["rows"][-1].float() - outs["rows_q"][-1].float()).abs().max() > 2e-2
    assert torch.allclose(outs["rows"][-1].float(), outs["rows_q"][-1].float(), atol=0.5)


def test_sampler_candidates_and_draw():
    """topk_probs against torch.topk + F.softmax; sample_topk against a brute-force float64 scan and, over many
    uniform numbers, against the probabilities themselves"""
    import torch.nn.functional as F
    g = torch.Generator().manual_seed(77)
    logits = (torch.randn((6, 500), generator=g) * 3).half()
    for temperature, k in ((1.0, 32), (0.7, 5), (2.5, 500)):
        p, idx = O.topk_probs(logits, temperature, k)
        v_ref, _ = torch.topk(logits / temperature, k)
        assert torch.equal(torch.gather(logits / temperature, 1, idx), v_ref)          # same values in the same order
        assert torch.equal(p, F.softmax(v_ref, dim=-1))
    # k = 1 is the argmax whatever u is
    u = torch.rand(6, generator=g)
    assert torch.equal(O.sample_topk(logits, 1.0, 1, u), logits.float().argmax(-1))
    # huge temperature, all candidates: uniform probabilities
    p, _ = O.topk_probs(logits, 1e4, 500)
    assert torch.allclose(p.float(), torch.full_like(p, 1 / 500).float(), rtol=2e-2)
    # the draw: brute force in float64
    p, idx = O.topk_probs(logits, 0.9, 20)
    for trial in range(50):
        u = torch.rand(6, generator=g)
        got = O.sample_topk(logits, 0.9, 20, u)
        for r in range(6):
            cum, pick = 0.0, 19
            tot = float(p[r].double().sum())
            for j in range(20):
                cum += float(p[r, j])
                if cum > float(u[r]) * tot + 1e-9:
                    pick = j
                    break
            near = abs(cum - float(u[r]) * tot) < 1e-5          # a boundary within fp32 rounding of the target
            assert int(got[r]) == int(idx[r, pick]) or near
    # frequencies over many draws follow p (row 0, 5 candidates)
    p, idx = O.topk_probs(logits[:1], 1.0, 5)
    n = 20000
    u = torch.rand(n, generator=g)
    draws = O.sample_topk(logits[:1].expand(n, -1).contiguous(), 1.0, 5, u)
    for j in range(5):
        freq = float((draws == idx[0, j]).float().mean())
        assert abs(freq - float(p[0, j])) < 4 * (float(p[0, j]) * (1 - float(p[0, j])) / n) ** 0.5 + 1e-3


def test_filter_sampler_keeps_every_value_equal_to_the_kth():
    """topk_filter_probs (hf_model_q40.py:521-529) against hand-computed cases and float64 properties: the support is
    exactly the values >= the k-th largest (brute-force count), probabilities are exp(x / T) over the support in float64;
    sample_topk_filter against a scalar float64 scan and the probabilities themselves"""
    import math
    # 3, 3, 2, 2, 2, 1 with k = 3: the k-th largest is 2, all three 2s stay
    row = torch.tensor([[2.0, 3.0, 1.0, 2.0, 3.0, 2.0]], dtype=torch.float16)
    p = O.topk_filter_probs(row, 1.0, 3)[0].double()
    z = 2 * math.exp(3) + 3 * math.exp(2)
    want = torch.tensor([math.exp(2) / z, math.exp(3) / z, 0.0, math.exp(2) / z, math.exp(3) / z, math.exp(2) / z], dtype=torch.float64)
    assert torch.allclose(p, want, rtol=1e-6, atol=0)
    # k = 2: the k-th largest is 3, only the two 3s
    p = O.topk_filter_probs(row, 0.5, 2)[0]
    assert p.tolist() == [0.0, 0.5, 0.0, 0.0, 0.5, 0.0]
    g = torch.Generator().manual_seed(78)
    logits = torch.round(torch.randn((5, 400), generator=g) * 6).half() / 2          # a coarse grid: many equal values
    for temperature, k in ((1.0, 32), (0.7, 5), (2.5, 400), (1.3, 1)):
        p = O.topk_filter_probs(logits, temperature, k)
        for r in range(5):
            vals = sorted(logits[r].tolist(), reverse=True)
            kth = vals[k - 1]
            support = [i for i in range(400) if float(logits[r, i]) >= kth]
            assert len(support) >= k and sorted((p[r] > 0).nonzero().flatten().tolist()) == support
            z = sum(math.exp((float(logits[r, i]) - vals[0]) / temperature) for i in support)
            for i in support[:50]:
                assert abs(float(p[r, i]) - math.exp((float(logits[r, i]) - vals[0]) / temperature) / z) < 1e-6
            assert abs(float(p[r].double().sum()) - 1.0) < 1e-5
    # the draw: scalar scan over (value descending, index ascending)
    p = O.topk_filter_probs(logits, 0.9, 20)
    for trial in range(30):
        u = torch.rand(5, generator=g)
        got = O.sample_topk_filter(logits, 0.9, 20, u)
        for r in range(5):
            order = sorted(range(400), key=lambda i: (-float(logits[r, i]), i))
            alive = [i for i in order if float(p[r, i]) > 0]
            tot = sum(float(p[r, i]) for i in alive)
            cum, pick, near = 0.0, alive[-1], False
            for i in alive:
                cum += float(p[r, i])
                near = near or abs(cum - float(u[r]) * tot) < 1e-5
                if cum > float(u[r]) * tot:
                    pick = i
                    break
            assert int(got[r]) == pick or near
    # frequencies over many draws follow p
    n = 20000
    u = torch.rand(n, generator=g)
    draws = O.sample_topk_filter(logits[:1].expand(n, -1).contiguous(), 1.0, 4, u)
    p = O.topk_filter_probs(logits[:1], 1.0, 4)[0]
    for i in (p > 0).nonzero().flatten().tolist():
        freq = float((draws == i).float().mean()); pi = float(p[i])
        assert abs(freq - pi) < 4 * (pi * (1 - pi) / n) ** 0.5 + 1e-3


TERMINAL = [29961, 29914, 20055, 4690, 1164, 29962]          # "[/PYTHON]" as the reference tokenises it (mcts.py:12)


def scalar_terminal_walk(tokens, seq, eos=2):
    """a branch's token stream, one token at a time, as plain control flow: returns (ended flags, states)"""
    ended, states, st = [], [], 0
    for tok in tokens:
        if tok == seq[st]:
            st += 1
        else:
            st = 0
        done = st == len(seq) or tok == eos
        if done:
            st = 0
        ended.append(done)
        states.append(st)
    return ended, states


def test_terminal_state_machine_known_answers_and_scalar_walk():
    seq = torch.tensor(TERMINAL, dtype=torch.int64)

    def run(tokens):
        st = torch.zeros(1, dtype=torch.int32)
        ended, states = [], []
        for tok in tokens:
            e, st = O.detect_terminal(torch.tensor([tok], dtype=torch.int64), st, seq)
            ended.append(bool(e[0]))
            states.append(int(st[0]))
        return ended, states

    # the sequence in order ends at its last token and the state restarts
    assert run(TERMINAL) == ([False] * 5 + [True], [1, 2, 3, 4, 5, 0])
    # end-of-sequence ends at once, from any state
    assert run([7, 2]) == ([False, True], [0, 0])
    assert run(TERMINAL[:3] + [2]) == ([False, False, False, True], [1, 2, 3, 0])
    # a wrong token resets; a repeated first token does not restart the match (the reference's transition)
    assert run(TERMINAL[:2] + [5] + TERMINAL) == ([False] * 8 + [True], [1, 2, 0, 1, 2, 3, 4, 5, 0])
    assert run([TERMINAL[0], TERMINAL[0], TERMINAL[1]])[1] == [1, 0, 0]
    # every (state, token class) pair: the expected token, another token of the sequence, a foreign token, eos
    for st0 in range(6):
        for tok in TERMINAL + [11, 2]:
            e, st = O.detect_terminal(torch.tensor([tok], dtype=torch.int64), torch.tensor([st0], dtype=torch.int32), seq)
            nxt = st0 + 1 if tok == TERMINAL[st0] else 0
            done = nxt == 6 or tok == 2
            assert (bool(e[0]), int(st[0])) == (done, 0 if done else nxt)
    # random streams with the sequence spliced in, batched, against the scalar walk
    g = torch.Generator().manual_seed(77)
    streams = []
    for b in range(16):
        toks = torch.randint(0, 40, (60,), generator=g).tolist()
        toks = [TERMINAL[t % 6] if t < 12 else t for t in toks]          # many near-matches
        at = int(torch.randint(0, 50, (1,), generator=g))
        toks[at:at + 6] = TERMINAL
        streams.append(toks[:60])
    st = torch.zeros(16, dtype=torch.int32)
    want = [scalar_terminal_walk(s_, TERMINAL) for s_ in streams]
    for i in range(60):
        e, st = O.detect_terminal(torch.tensor([s_[i] for s_ in streams], dtype=torch.int64), st, seq)
        assert e.tolist() == [w[0][i] for w in want]
        assert st.tolist() == [w[1][i] for w in want]


def test_noise_study_instruments_reduce_to_the_oracle_where_they_must():
    """The oracle's noise-study switches (double-precision accumulation, scale on the activation side, fp16 prefix
    probabilities, fp16 K-slice partial sums) change WHERE a rounding happens, never the value before rounding: each
    must reproduce the plain oracle on inputs where that rounding is exact, and stay within fp16 noise otherwise."""
    cfg = dict(dim=256, n_layers=2, n_heads=2, vocab_size=320, multiple_of=128, max_batch_size=2, max_seq_len=8, max_prompt_seq_len=16)
    args = O.OracleArgs(**cfg)
    sd = O.random_q40_state_dict(args, seed=70, std=0.05)
    g = torch.Generator().manual_seed(71)
    prompt = torch.randint(0, 320, (1, 12), generator=g)
    base = O.OracleTransformer(args, sd, dense=True)
    toks, _ = base.greedy(prompt, 1, 6)
    want = base.forced(prompt, toks[0])
    assert want.shape == (6, 320)
    assert torch.equal(want.argmax(-1), toks[0])                      # forced on its own tokens = its greedy run
    # one K-slice: the fp16 rounding of the only partial sum is the result's own rounding
    one = O.OracleTransformer(args, sd, dense=True, slab_half_ksplit=lambda key, K, N: 1, share_dense=base)
    assert torch.equal(one.forced(prompt, toks[0]), want)
    # several slices, double precision: close, not necessarily equal
    for kw in (dict(slab_half_ksplit=lambda key, K, N: 4, share_dense=base), dict(acc_dtype=torch.float64), dict(p_half_prefix=True, share_dense=base),
               dict(scale_on_x_max_rows=16, share_dense=base)):
        got = O.OracleTransformer(args, sd, dense=True, **kw).forced(prompt, toks[0])
        assert torch.allclose(got, want, rtol=0, atol=0.05) and float((got - want).abs().max()) > 0.0, kw
    # power-of-two scales: x * scale and code * scale are both exact in fp16, so moving the rounding changes nothing
    # (double-precision accumulation on both sides, so that the summation order does not matter either)
    sd2 = dict(sd)
    for k in list(sd2):
        if k.endswith(".s"):
            s = sd2[k].float()
            sd2[k] = torch.where(s > 0, torch.exp2(torch.round(torch.log2(s.clamp_min(1e-8)))), s).to(torch.float16)
    a64 = O.OracleTransformer(args, sd2, dense=True, acc_dtype=torch.float64)
    b64 = O.OracleTransformer(args, sd2, dense=True, acc_dtype=torch.float64, scale_on_x_max_rows=16)
    x = ((torch.rand((3, 256), generator=g) * 1.9 + 0.1) * torch.where(torch.rand((3, 256), generator=g) < 0.5, -1.0, 1.0)).half()    # no product underflows
    for key in ("layers.0.attention.wq", "layers.1.feed_forward.w1"):
        assert torch.equal(a64._linear(key, x), b64._linear(key, x))
    x20 = torch.cat([x] * 7)[:20]                                     # 20 rows: above the limit, the dense path in both
    assert torch.equal(a64._linear("layers.0.attention.wo", x20), b64._linear("layers.0.attention.wo", x20))
    # uniform scores: every prefix probability is exp(0) = 1, exact in fp16
    q = torch.zeros((2, 2, 128), dtype=torch.float16)
    pk, pv = torch.randn((9, 2, 128), generator=g).half(), torch.randn((9, 2, 128), generator=g).half()
    sk, sv = torch.randn((2, 3, 2, 128), generator=g).half(), torch.randn((2, 3, 2, 128), generator=g).half()
    assert torch.equal(O.shared_prefix_attention(q, pk, pv, sk, sv, [3, 1], p_half_prefix=True), O.shared_prefix_attention(q, pk, pv, sk, sv, [3, 1]))
    qq = torch.randn((2, 2, 128), generator=g).half()
    d = (O.shared_prefix_attention(qq, pk, pv, sk, sv, [3, 1], p_half_prefix=True).float() - O.shared_prefix_attention(qq, pk, pv, sk, sv, [3, 1]).float()).abs().max()
    assert float(d) <= 2e-3
    d = (O.shared_prefix_attention(qq, pk, pv, sk, sv, [3, 1], acc_dtype=torch.float64).float() - O.shared_prefix_attention(qq, pk, pv, sk, sv, [3, 1]).float()).abs().max()
    assert float(d) <= 2e-3


def test_row_temperature_known_answers():
    """The temp <= 0 mode of the tree sampler (mcts.py:110-114): the ramp's end points, and draws whose probabilities are
    worked out by hand.  Two candidates with logits (0, T ln 3) at temperature T have probabilities (1/4, 3/4); in
    descending order the cumulative sums are (3/4, 1): a uniform number below 3/4 picks the larger logit."""
    counts = torch.tensor([1, 12, 4], dtype=torch.int32)
    t = O.ramp_temperature(-0.7, 12, counts)
    assert t.dtype == torch.float32
    assert float(t[0]) == pytest.approx(0.1, abs=1e-7) and float(t[1]) == pytest.approx(0.7, abs=1e-6)
    assert float(t[2]) == pytest.approx(0.1 + 0.6 * 3 / 11, abs=1e-6)
    assert torch.equal(O.ramp_temperature(0.7, 12, counts), t)                 # the sign only selects the mode
    ln3 = 1.0986328125                                                        # fp16(ln 3)
    logits = torch.full((2, 8), -30.0, dtype=torch.float16)
    logits[:, 5] = 0.0
    logits[0, 2] = 0.5 * ln3                                                  # row 0 at T = 0.5
    logits[1, 2] = 0.5 * ln3                                                  # row 1 at T = 1: p = (0.634, 0.366)
    temps = torch.tensor([0.5, 1.0])
    p, order = O.topk_probs(logits, temps, 2)
    assert p.dtype == torch.float32 and order.tolist() == [[2, 5], [2, 5]]
    assert float(p[0, 0]) == pytest.approx(0.75, abs=2e-4) and float(p[1, 0]) == pytest.approx(3 ** 0.5 / (1 + 3 ** 0.5), abs=2e-4)
    u = torch.tensor([0.70, 0.80, 0.60, 0.70])
    got = O.sample_topk_counts(logits, temps, 2, [2, 2], u)
    assert got.tolist() == [2, 5, 2, 5]                                       # row 0: 0.70 < 3/4 <= 0.80; row 1: 0.60 < 0.634 <= 0.70
    # a scalar temperature keeps the fp16 path: same candidates, probabilities rounded to fp16
    p16, order16 = O.topk_probs(logits[:1], 0.5, 2)
    assert p16.dtype == torch.float16 and order16.tolist() == [[2, 5]] and float(p16[0, 0]) == pytest.approx(0.75, abs=1e-3)


def test_tree_fork_known_answers():
    """The expansion bookkeeping of the tree sampler (mcts.py:127-152) on a tree small enough to write every row out by hand."""
    B, steps = 6, 4
    results = torch.zeros((B, steps), dtype=torch.int64)
    results[0, 0], results[1, 0] = 11, 12
    oc = torch.zeros((2, B), dtype=torch.int32)
    oc[0, 0], oc[1, 0], oc[0, 1], oc[1, 1] = 11, 4, 12, 2
    alive = torch.tensor([True, True, True, True, True, True])
    pages = torch.arange(B * 5, dtype=torch.int32).view(B, 5)
    # branch 0 drew 7, 5, 7, 9 -> distinct 5 (x1), 7 (x2), 9 (x1); branch 1 drew 3, 3 -> distinct 3 (x2)
    draws = torch.tensor([7, 5, 7, 9, 3, 3])
    cur, origin = O.tree_fork(draws, oc, alive, 2, B, results, 1, pages, n_rows=2)
    assert cur == 4 and origin == [-1, -1, 0, 0, -1, -1]
    assert results[:, :2].tolist() == [[11, 5], [12, 3], [11, 7], [11, 9], [0, 0], [0, 0]]
    assert oc.tolist() == [[5, 3, 7, 9, 0, 0], [1, 2, 2, 1, 0, 0]] and int(oc[1].sum()) == 6       # multiplicities conserved
    assert pages[2, :2].tolist() == pages[0, :2].tolist() == [0, 1] and pages[2, 2:].tolist() == [12, 13, 14]
    assert pages[3, :2].tolist() == [0, 1]
    # next step: branch 1 is dead (its draws change nothing, its column is zeroed), branch 2 forks once more
    alive = torch.tensor([True, False, True, True, True, True])
    draws = torch.tensor([8,   4, 4,   6, 2,   1])       # branch 0: 8 | branch 1: 4 4 | branch 2: 6 2 | branch 3: 1
    oc2 = oc.clone()
    cur, origin = O.tree_fork(draws, oc2, alive, 4, B, results, 2, pages, n_rows=3)
    assert cur == 5 and origin == [-1, -1, -1, -1, 2, -1]
    assert results[:, :3].tolist() == [[11, 5, 8], [12, 3, 0], [11, 7, 2], [11, 9, 1], [11, 7, 6], [0, 0, 0]]
    assert oc2[0].tolist() == [8, 3, 2, 1, 6, 0] and oc2[1].tolist() == [1, 2, 1, 1, 1, 0]
    assert pages[4, :3].tolist() == pages[2, :3].tolist() == [0, 1, 12] and pages[4, 3:].tolist() == [23, 24]
    # rows run out: branch 0 draws three distinct tokens with one row left; the last distinct token and its multiplicity
    # are dropped, as in the reference (forks = min(len(counts) - 1, batch_size - curr_batch_size), mcts.py:141-142)
    r4 = torch.zeros((3, 2), dtype=torch.int64)
    oc4 = torch.tensor([[0, 0, 0], [3, 1, 0]], dtype=torch.int32)
    cur, origin = O.tree_fork(torch.tensor([7, 5, 6, 9]), oc4, torch.ones(3, dtype=torch.bool), 2, 3, r4, 0)
    assert cur == 3 and origin == [-1, -1, 0] and r4[:, 0].tolist() == [5, 9, 6] and oc4.tolist() == [[5, 9, 6], [1, 1, 1]]
    # a full tree: nothing forks any more
    alive6 = torch.ones(6, dtype=torch.bool)
    oc3 = torch.tensor([[0] * 6, [1, 1, 1, 1, 1, 1]], dtype=torch.int32)
    r3 = torch.zeros((6, 2), dtype=torch.int64)
    cur, origin = O.tree_fork(torch.arange(6) + 20, oc3, alive6, 6, 6, r3, 0)
    assert cur == 6 and origin == [-1] * 6 and r3[:, 0].tolist() == [20, 21, 22, 23, 24, 25]
    # draws per row against the single-draw sampler
    g = torch.Generator().manual_seed(5)
    logits = torch.randn((3, 50), generator=g).half()
    u = torch.rand(7, generator=g)
    got = O.sample_topk_counts(logits, 0.7, 8, [2, 0, 5], u)
    want = torch.cat([O.sample_topk(logits[0:1].expand(2, -1), 0.7, 8, u[:2]), O.sample_topk(logits[2:3].expand(5, -1), 0.7, 8, u[2:])])
    assert torch.equal(got, want)
