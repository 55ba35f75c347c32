#!/usr/bin/env python3
"""Writes the fixture tests/golden/greedy_7b.json: the oracle's greedy tokens for the 7B-architecture random-init
Q4_0 model (BASELINE configs[3]: 32 layers, dim 4096, 32 heads, FFN 11008, vocab 32016, RoPE theta 1e6, 512-token
prompt), 64 steps at B=1, their top-1/top-2 logit margins, and a noise study that says which of those margins an
implementation can be held to.

The noise study runs the oracle again, teacher-forced on its own tokens, with ONE rounding moved each time (the
switches of oracle.q40_oracle.OracleTransformer) and records per step how far the logits move:
  acc64      every product and the attention accumulated in double precision: the distance between two faithful
             evaluations of the reference's cast points.  near_tie is derived from this run alone.
  scale_on_x the linears of the decode steps round fp16(x * scale) instead of fp16(code * scale)   (the GPU's GEMV)
  p_half     the prefix keys' probabilities rounded to fp16 before they multiply V                 (matrix-core P.V)
  slab_half  K-slice partial sums rounded to fp16 before they are added, slices as the GPU's GEMM
             cuts them at 100 rows                                                                 (the GPU's GEMM above 16 rows)
near_tie = 2 x the largest change of the top-1/top-2 gap between the fp32 and the fp64 oracle: a step whose margin is
below it can be decided either way by implementations that both follow the reference exactly.

Needs a GPU (the weights are generated and quantised there by bench.build_model, then copied to the host) and about
90 GB of host memory.  Run from the repository root on the GPU box; results land in greedy_7b.json next to this
script and in the run's output folder (OUT_DIR below):

    python tests/golden/make_7b_greedy.py [--seed 3] [--variants acc64,scale_on_x,p_half,slab_half]

With --variants given and tests/golden/greedy_7b.json present for the same seed, only those studies are (re)run and
merged into it.
"""
import argparse
import gc
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
OUT_DIR = "gpurun_out"
sys.path.insert(0, ROOT)
import bench                                  # noqa: E402  (build_model: the generator of the 7B random weights)
from oracle import q40_oracle as O            # noqa: E402

ARGS = dict(dim=4096, n_layers=32, n_heads=32, vocab_size=32016, multiple_of=256, norm_eps=1e-5, rope_theta=1e6,
            max_batch_size=16, max_seq_len=128, max_prompt_seq_len=512)
STEPS = 64
PROMPT = 512
ALL = ("acc64", "scale_on_x", "p_half", "slab_half")
T0 = time.time()


def heartbeat():
    import threading

    def beat():
        while True:
            time.sleep(30)
            print(f"  ... {time.time() - T0:.0f} s", flush=True)
    threading.Thread(target=beat, daemon=True).start()


def gemm_ksplit_at_100_rows(key, K, N):
    """K-slices of the GPU's GEMM at M = 100 for the launches of a 7B decode layer: wq|wk|wv (48 column units) and
    w1|w3 (86) take 5, the 4096-wide wo and w2 (16 units) take 16."""
    return 16 if key.endswith(("attention.wo", "feed_forward.w2")) else 5


def study(name, args, sd, prompt, tokens, base_logits, share):
    kw = {"acc64": dict(acc_dtype=torch.float64), "scale_on_x": dict(scale_on_x_max_rows=16, share_dense=share),
          "p_half": dict(p_half_prefix=True, share_dense=share),
          "slab_half": dict(slab_half_ksplit=gemm_ksplit_at_100_rows, share_dense=share)}[name]
    t0 = time.time()
    model = O.OracleTransformer(args, sd, dense=True, **kw)
    print(f"[{name}] oracle ready after {time.time() - t0:.0f} s", flush=True)
    logits = model.forced(prompt, tokens)
    del model
    gc.collect()
    top2 = base_logits.topk(2, dim=-1).indices                                  # the base oracle's two candidates per step
    gap_base = base_logits.gather(1, top2)[:, 0] - base_logits.gather(1, top2)[:, 1]
    gap_var = logits.gather(1, top2)[:, 0] - logits.gather(1, top2)[:, 1]
    out = {"max_abs_logit_diff": [round(float(x), 5) for x in (logits - base_logits).abs().max(dim=1).values],
           "gap_shift": [round(float(x), 5) for x in (gap_var - gap_base).abs()],
           "argmax_differs_at": [int(i) for i in torch.nonzero(logits.argmax(-1) != tokens).flatten()]}
    print(f"[{name}] done after {time.time() - t0:.0f} s: max |dlogit| {max(out['max_abs_logit_diff']):.4f}, max gap shift "
          f"{max(out['gap_shift']):.4f}, argmax differs at steps {out['argmax_differs_at']}", flush=True)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--seed", type=int, default=3)
    ap.add_argument("--variants", default=",".join(ALL))
    a = ap.parse_args()
    variants = [v for v in a.variants.split(",") if v]
    assert all(v in ALL for v in variants), variants
    heartbeat()
    seed = a.seed
    torch.manual_seed(seed)
    model = bench.build_model(torch, ARGS, seed=seed)
    prompt = torch.randint(0, ARGS["vocab_size"], (1, PROMPT), generator=torch.Generator().manual_seed(seed))
    sd = {"tok_embeddings.weight": model.tok_embeddings.weight.detach().cpu(), "output.weight": model.output.weight.detach().cpu(),
          "norm.weight": model.norm.weight.detach().cpu()}
    for i, layer in enumerate(model.layers):
        p = f"layers.{i}."
        sd[p + "attention_norm.weight"] = layer.attention_norm.weight.detach().cpu()
        sd[p + "ffn_norm.weight"] = layer.ffn_norm.weight.detach().cpu()
        for blk, names in (("attention", ("wq", "wk", "wv", "wo")), ("feed_forward", ("w1", "w2", "w3"))):
            for name in names:
                lin = getattr(getattr(layer, blk), name)
                sd[p + f"{blk}.{name}.w"] = lin.w.cpu()
                sd[p + f"{blk}.{name}.s"] = lin.s.cpu()
                sd[p + f"{blk}.{name}.shape"] = torch.Size((lin.shape[0], lin.shape[1]))     # (out, in), as the converter stores it
    del model
    torch.cuda.empty_cache()
    print(f"weights on the host after {time.time() - T0:.0f} s; building the dense oracle", flush=True)
    oargs = O.OracleArgs(**ARGS)
    base = O.OracleTransformer(oargs, sd, dense=True)
    print(f"oracle ready after {time.time() - T0:.0f} s; prefill + {STEPS} steps", flush=True)
    tokens, margins = base.greedy(prompt, 1, STEPS)
    tokens = tokens[0]
    print(f"greedy run done after {time.time() - T0:.0f} s; min margin {min(margins):.4f}", flush=True)
    path = os.path.join(ROOT, "tests", "golden", "greedy_7b.json")
    out = {"seed": seed, "prompt_len": PROMPT, "steps": STEPS, "args": ARGS,
           "tokens": tokens.tolist(), "margins": [round(m, 5) for m in margins], "noise": {}}
    if os.path.exists(path):
        old = json.load(open(path))
        if old.get("seed") == seed:
            assert old["tokens"] == out["tokens"], "the oracle's tokens changed for the same seed"
            out["noise"] = old.get("noise", {})
    if variants:
        base_logits = base.forced(prompt, tokens)
        assert torch.equal(base_logits.argmax(-1), tokens)
        print(f"forced base run done after {time.time() - T0:.0f} s", flush=True)
        for name in [v for v in variants if v != "acc64"]:
            out["noise"][name] = study(name, oargs, sd, prompt, tokens, base_logits, base)
        del base
        gc.collect()
        if "acc64" in variants:
            out["noise"]["acc64"] = study("acc64", oargs, sd, prompt, tokens, base_logits, None)
    if "acc64" in out["noise"]:
        out["near_tie"] = round(2.0 * max(out["noise"]["acc64"]["gap_shift"]), 5)
    os.makedirs(os.path.join(ROOT, OUT_DIR), exist_ok=True)
    for dst in (path, os.path.join(ROOT, OUT_DIR, "greedy_7b.json")):
        with open(dst, "w") as f:
            json.dump(out, f)
    print(json.dumps({k: v for k, v in out.items() if k != "noise"})[:600])
    print("near_tie", out.get("near_tie"), "steps below it:", sum(m < out.get("near_tie", 0) for m in margins))


if __name__ == "__main__":
    main()
