#!/usr/bin/env python3
"""Writes tests/golden/greedy_7b.json: the oracle's greedy tokens and top-1/top-2 logit margins for the
7B-architecture random-init Q4_0 model (BASELINE configs[3]: 32 layers, dim 4096, 32 heads, FFN 11008,
vocab 32016, RoPE theta 1e6, 512-token prompt), 64 decode steps at B=1.

Needs a GPU (the weights are generated and quantised there, by the same generator bench.py uses, and
copied to the host for the oracle) and about 60 GB of host memory: the oracle runs the dense fp32
restatement of the model on the CPU.  Takes a few minutes; run from the repository root:

    python tests/golden/make_7b_greedy.py [seed]

The test that consumes the fixture (tests/test_gpu_model_7b.py) regenerates the same weights from
the seed and feeds the ORACLE's tokens to the GPU model step by step, so one near-tie does not hide
the steps after it.
"""
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import bench                                  # noqa: E402  (build_model: the generator of the 7B random weights)
from oracle import q40_oracle as O            # noqa: E402

ARGS = dict(dim=4096, n_layers=32, n_heads=32, vocab_size=32016, multiple_of=256, norm_eps=1e-5, rope_theta=1e6,
            max_batch_size=16, max_seq_len=128, max_prompt_seq_len=512)
STEPS = 64
PROMPT = 512


def heartbeat():
    import threading

    def beat():
        t0 = time.time()
        while True:
            time.sleep(30)
            print(f"  ... {time.time() - t0:.0f} s", flush=True)
    threading.Thread(target=beat, daemon=True).start()


def main():
    heartbeat()
    seed = int(sys.argv[1]) if len(sys.argv) > 1 else 3
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
    print("weights on the host; building the dense oracle", flush=True)
    t0 = time.time()
    oargs = O.OracleArgs(**ARGS)
    oracle = O.OracleTransformer(oargs, sd, dense=True)
    print(f"oracle ready after {time.time() - t0:.0f} s; prefill + {STEPS} steps", flush=True)
    tokens, margins = oracle.greedy(prompt, 1, STEPS)
    print(f"done after {time.time() - t0:.0f} s; min margin {min(margins):.4f}", flush=True)
    out = {"seed": seed, "prompt_len": PROMPT, "steps": STEPS, "args": ARGS,
           "tokens": tokens[0].tolist(), "margins": [round(m, 5) for m in margins]}
    with open(os.path.join(ROOT, "tests", "golden", "greedy_7b.json"), "w") as f:
        json.dump(out, f)
    print(json.dumps(out)[:400])


if __name__ == "__main__":
    main()
