"""Greedy decoding of the 7B-architecture random-init Q4_0 model (BASELINE configs[3]) against the oracle's tokens held
in tests/golden/greedy_7b.json (made by tests/golden/make_7b_greedy.py: dense fp32 CPU restatement of the model on the
same generated weights, plus a noise study).

Every path the benchmark times is held against the fixture: one branch (tiled GEMV with the RMSNorm and SiLU made inside
the matmul launches, the one-launch attention), ten branches (GEMV, separate small kernels) and a hundred (the MFMA
GEMM, the two-launch attention).  Two runs per path:
  teacher-forced  the GPU model is fed the ORACLE's previous token, so each of the 64 steps is checked on its own.  A step
                  may differ only where the oracle itself cannot decide it: its top-1/top-2 margin there is at most twice
                  what the same oracle accumulating in double precision moves that margin AT THAT STEP, or one fp16 ulp of
                  the logit (two faithful evaluations of the reference's cast points drift that far apart on this chaotic
                  32-layer random model).  At most one of the 64 steps may differ per path.
  free-running    the GPU model is fed its own tokens, as the benchmark runs it; the common prefix with the oracle's tokens
                  must reach the path's first differing teacher-forced step (all 64 tokens when none differs).
The per-path lines (matches, differing steps with their margins and bounds, free-run length) are also written to
greedy_7b_paths.md in the run's output folder (REPORT_DIR below)."""
import json
import os

REPORT_DIR = "gpurun_out"

import pytest
import torch

pytestmark = pytest.mark.gpu

FIXTURE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "greedy_7b.json")


def _fp16_ulp(x: float) -> float:
    import math
    x = abs(float(x))
    return 2.0 ** (max(math.floor(math.log2(x)), -14) - 10) if x > 0 else 2.0 ** -24


def test_7b_greedy_tokens_match_oracle():
    import bench
    from spec_mcts_amd import kernels as K
    fx = json.load(open(FIXTURE))
    seed, P, steps = fx["seed"], fx["prompt_len"], fx["steps"]
    assert fx["near_tie"] == pytest.approx(2.0 * max(fx["noise"]["acc64"]["gap_shift"]), abs=1e-4)
    want = torch.tensor(fx["tokens"], dtype=torch.int64)
    margins, shift64 = fx["margins"], fx["noise"]["acc64"]["gap_shift"]
    torch.manual_seed(seed)
    model = bench.build_model(torch, dict(fx["args"], max_batch_size=100), seed=seed)
    prompt = torch.randint(0, fx["args"]["vocab_size"], (1, P), generator=torch.Generator().manual_seed(seed)).cuda()
    report = ["# Greedy tokens of the 7B-architecture model against the oracle's (tests/test_gpu_model_7b.py)\n",
              f"Fixture: seed {seed}, {P}-token prompt, {steps} greedy steps; smallest oracle margins: "
              + ", ".join(f"step {i}: {margins[i]}" for i in sorted(range(steps), key=lambda i: margins[i])[:4]) + ".\n",
              "| branches | teacher-forced equal | differing steps (oracle margin, bound) | free-running equal |", "|---:|---:|---|---:|"]
    for B in (1, 10, 100):
        # ---- teacher-forced ----
        model.resetSeq()
        logits = model(prompt, 0)[:, -1]
        got = torch.zeros((B, steps), dtype=torch.int64)
        top = torch.zeros(steps)
        got[:, 0] = int(K.argmax(logits.contiguous())[0])
        top[0] = float(logits[0].max())
        for s in range(1, steps):
            tok = want[s - 1].expand(B, 1).contiguous().cuda()            # the oracle's token, not the model's own
            lg = model(tok, P + s - 1)[:, -1]
            got[:, s] = K.argmax(lg.contiguous()).cpu()
            top[s] = float(lg[0].max())
        torch.cuda.synchronize()
        for b in range(1, B):
            assert torch.equal(got[b], got[0]), "identical branches must produce identical tokens"
        differing = [i for i in range(steps) if int(got[0, i]) != int(want[i])]
        bound = {i: max(2.0 * shift64[i], _fp16_ulp(top[i])) for i in differing}
        print(f"B={B} teacher-forced: {steps - len(differing)}/{steps} tokens equal the oracle's; differing steps (oracle margin, bound) "
              f"{[(i, margins[i], bound[i]) for i in differing]}", flush=True)
        # ---- free-running ----
        model.resetSeq()
        logits = model(prompt, 0)[:, -1]
        free = torch.zeros((B, steps), dtype=torch.int64, device="cuda:0")
        free[:, 0] = K.argmax(logits.contiguous())[0]
        for s in range(1, steps):
            lg = model(free[:, s - 1:s].contiguous(), P + s - 1)[:, -1]
            free[:, s] = K.argmax(lg.contiguous())
        free = free.cpu()
        for b in range(1, B):
            assert torch.equal(free[b], free[0])
        run = next((i for i in range(steps) if int(free[0, i]) != int(want[i])), steps)
        print(f"B={B} free-running: first {run} tokens equal the oracle's" + (f" (oracle margin at step {run}: {margins[run]})" if run < steps else ""), flush=True)
        report.append(f"| {B} | {steps - len(differing)} / {steps} | " + (", ".join(f"step {i} ({margins[i]}, {bound[i]:.4f})" for i in differing) or "none")
                      + f" | {run} / {steps} |")
        _write_report(report)
        wrong = [i for i in differing if margins[i] > bound[i]]
        assert not wrong, f"B={B}: tokens differ at steps {wrong} where the oracle's margin {[margins[i] for i in wrong]} exceeds {[bound[i] for i in wrong]}"
        assert len(differing) <= 1, f"B={B}: {len(differing)} of {steps} teacher-forced tokens differ from the oracle's (at most one may)"
        first_diff = differing[0] if differing else steps
        assert run >= first_diff, f"B={B}: free-running tokens leave the oracle's at step {run}, before the first undecidable step ({first_diff})"


def _write_report(lines):
    out = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), REPORT_DIR)
    try:
        os.makedirs(out, exist_ok=True)
        with open(os.path.join(out, "greedy_7b_paths.md"), "w") as f:
            f.write("\n".join(lines) + "\n")
    except OSError:
        pass


@pytest.mark.parametrize("batch_size", [80, 100])
def test_7b_tree_search_at_full_size(batch_size):
    """mcts.search on the 7B architecture with a 512-token prompt at the reference's batch sizes (load_q40.py:183: up to
    80; infer_code.py:157: 100): the loop's own invariants (mcts.py:154-155: never more than batch_size branches, the
    multiplicities add up to batch_size), the tree structure of the returned rows, and the same tokens from the search
    whose steps replay HIP graphs and from the one that issues every launch."""
    import bench
    from spec_mcts_amd.mcts import mcts
    fx = json.load(open(FIXTURE))
    seed, P = fx["seed"], fx["prompt_len"]
    torch.manual_seed(seed)
    model = bench.build_model(torch, dict(fx["args"], max_batch_size=100), seed=seed)
    prompt = torch.randint(0, fx["args"]["vocab_size"], (1, P), generator=torch.Generator().manual_seed(seed)).cuda()
    depth = 24
    runs = []
    for use_graph in (True, False):
        tree = mcts(model, depth, top_k=32, temp=0.8)
        tree.use_graph = use_graph
        tree.generator = torch.Generator(device="cuda:0").manual_seed(77)
        res, res_len, stats = tree.search(prompt, batch_size)
        torch.cuda.synchronize()
        stats, res_c = stats.cpu().tolist(), res.cpu()
        curr = res.shape[0]
        assert curr <= batch_size and curr == stats[-1]
        assert all(a <= b for a, b in zip(stats, stats[1:])), "the number of branches never shrinks"
        counts = tree.last_counts.cpu()
        assert int(counts[1].sum()) == batch_size and bool((counts[1, :curr] >= 1).all()) and bool((counts[1, curr:] == 0).all())
        assert tree.last_replays == (tree.last_steps if use_graph else 0)
        assert curr > 1, "the tree did not branch"
        # row r was created at the first step whose branch count exceeds r: up to there it repeats an earlier row, at that
        # step it takes another token than that row
        for r in range(1, curr):
            born = next(t for t, c in enumerate(stats) if c > r)
            assert any(torch.equal(res_c[r, :born], res_c[o, :born]) and int(res_c[r, born]) != int(res_c[o, born]) for o in range(r)), r
        # lengths: a live row has one token per step
        assert int(res_len.max()) <= res.shape[1]
        runs.append((res_c, res_len.cpu(), stats))
    if batch_size <= 16:
        assert torch.equal(runs[0][0], runs[1][0])
    assert runs[0][2][-1] == batch_size or len(runs[0][2]) == depth
