"""Greedy decoding of the 7B-architecture random-init Q4_0 model (BASELINE configs[3]) against the oracle's
tokens held in tests/golden/greedy_7b.json (made by tests/golden/make_7b_greedy.py: dense fp32 CPU
restatement of the model on the same generated weights).

The GPU model is fed the ORACLE's previous token at every step (teacher forcing), so each of the 64 steps
is checked on its own: a step counts when the oracle's top-1/top-2 logit margin is above NEAR_TIE; below
it the argmax is decided by rounding noise and the step is only reported.

How large that noise is was measured, not guessed: this random-init model is chaotic (32 layers of random
weights and Q4_0-quantised KV rows), and the two GPU paths of this package - the persistent step kernel and
the operator kernels, which round at the same points and differ ONLY in the order of fp32 partial sums -
disagree by 0.03 to 0.09 in the largest logit difference of a step (logits are fp16 numbers up to 6.5, one
ulp is 0.004 to 0.008).  NEAR_TIE is set to the top of that band."""
import json
import os

import pytest
import torch

pytestmark = pytest.mark.gpu

NEAR_TIE = 0.09
FIXTURE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "greedy_7b.json")


def test_7b_greedy_tokens_match_oracle():
    import bench
    from spec_mcts_amd import kernels as K
    fx = json.load(open(FIXTURE))
    seed, P, steps = fx["seed"], fx["prompt_len"], fx["steps"]
    want = torch.tensor(fx["tokens"], dtype=torch.int64)
    margins = fx["margins"]
    torch.manual_seed(seed)
    model = bench.build_model(torch, fx["args"], seed=seed)
    prompt = torch.randint(0, fx["args"]["vocab_size"], (1, P), generator=torch.Generator().manual_seed(seed)).cuda()
    decidable = [i for i, m in enumerate(margins) if m >= NEAR_TIE]
    assert len(decidable) >= steps * 2 // 3, "fixture has too many near-ties to be a test"
    for B in (1, 3, 10):
        print(f"B={B}", flush=True)
        model.resetSeq()
        logits = model(prompt, 0)[:, -1]
        got = torch.zeros((B, steps), dtype=torch.int64)
        got[:, 0] = int(K.argmax(logits.contiguous())[0])
        gaps = []
        for s in range(1, steps):
            tok = want[s - 1].expand(B, 1).contiguous().cuda()            # the oracle's token, not the model's own
            lg = model(tok, P + s - 1)[:, -1]
            got[:, s] = K.argmax(lg.contiguous()).cpu()
            top2 = lg[0].float().topk(2).values
            gaps.append(float(top2[0] - top2[1]))
        torch.cuda.synchronize()
        for b in range(1, B):
            assert torch.equal(got[b], got[0]), "identical branches must produce identical tokens"
        wrong = [i for i in decidable if int(got[0, i]) != int(want[i])]
        free_run = next((i for i in range(steps) if int(got[0, i]) != int(want[i])), steps)
        print(f"  matches {int((got[0] == want).sum())}/{steps}; decidable {len(decidable)}; first difference at step {free_run}; "
              f"oracle margins at differing steps {[margins[i] for i in range(steps) if int(got[0, i]) != int(want[i])]}", flush=True)
        assert not wrong, f"tokens differ at steps {wrong} where the oracle's margin is {[margins[i] for i in wrong]}"
