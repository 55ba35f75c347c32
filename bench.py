#!/usr/bin/env python3
"""Benchmark of the Q4_0 CodeLlama-7B-architecture decode hot path on one MI355X.

Workload (BASELINE.json configs[3]): random-init 7B architecture (32 layers, dim 4096, 32 heads,
FFN 11008, vocab 32016), weights ~N(0,0.02) in Q4_0, fp16 embeddings and lm_head; one 512-token
prompt prefilled once, then greedy decode with B = 1 / 10 / 100 branches sharing the prompt KV.
A "step" is one decode step (one new token per branch) through all layers, lm_head and argmax.

Prints ONE JSON line.  `value` is decode tokens/s at B=100 (all three batch sizes are in
`by_batch`); `roofline` describes the dominant kernel, the Q4_0 GEMV, timed live with HIP events
over one decode step's worth of weight matrices (224 distinct matrices, 3.44 GB, far larger than
the 256 MB Infinity Cache); `cpu_baseline` is the reference's CPU path (torch dequantise +
F.linear per linear, explicit softmax attention) timed on this box's host cores on one layer and
scaled to the model.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
PROMPT_LEN = 512
BATCHES = (1, 10, 100)
# architectures of the reference's checkpoints (params.json of CodeLlama-7b and -70b); "70b" is the one-GPU 70B
# workload: 2048-token prompt shared by the branches, 64 tokens decoded per branch
ARCHS = {
    "7b": dict(dim=4096, n_layers=32, n_heads=32, n_kv_heads=None, vocab_size=32016, multiple_of=256, ffn_dim_multiplier=None,
               prompt=PROMPT_LEN, max_seq_len=128),
    "70b": dict(dim=8192, n_layers=80, n_heads=64, n_kv_heads=8, vocab_size=32016, multiple_of=4096, ffn_dim_multiplier=1.3,
                prompt=2048, max_seq_len=64),
}
# HBM bytes per q40_gemv_kernel launch at M=1: rocprofv3 FETCH_SIZE + WRITE_SIZE, each scaled by a 1 GiB copy
# (profiles/q40_gemv_m1_hbm_traffic.md has the commands and the factors: 2.0 for reads, 1.0 for writes)
GEMV_TRAFFIC_BYTES_PER_LAUNCH = 27457381
# the same for the GEMM kernels at M=100 (profiles/q40_gemm_m100_hbm_traffic.md): 39.68 MB read + 8.47 MB written
# (the fp32 partial sums of the K-slices and the activations of w2 are the writes)
GEMM_TRAFFIC_BYTES_PER_LAUNCH = 48156518
# the same for one call of the decode attention leg (profiles/attn_decode_hbm_traffic.md): 65.6 MB read + 9.0 MB written
ATTN_TRAFFIC_BYTES_PER_CALL = 74610046


def q40_bytes(M, N, K):
    """algorithmic bytes of one Q4_0 matmul: packed nibbles + fp16 scales + activations + outputs"""
    return N * K // 2 + 2 * N * K // 64 + 2 * M * K + 2 * M * N


def build_model(torch, args_kw, seed):
    """Random-init Q4_0 model generated on the GPU (the host cannot hold or quantise 7B quickly)."""
    from spec_mcts_amd import ModelArgs, Transformer, kernels as K
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(seed)
    params = ModelArgs(**args_kw)
    model = Transformer(params)
    sd = {"tok_embeddings.weight": (torch.randn((params.vocab_size, params.dim), device=dev, generator=g) * 0.02).half(),
          "output.weight": (torch.randn((params.vocab_size, params.dim), device=dev, generator=g) * 0.02).half(),
          "norm.weight": torch.ones(params.dim, device=dev, dtype=torch.float16)}
    for i in range(params.n_layers):
        sd[f"layers.{i}.attention_norm.weight"] = torch.ones(params.dim, device=dev, dtype=torch.float16)
        sd[f"layers.{i}.ffn_norm.weight"] = torch.ones(params.dim, device=dev, dtype=torch.float16)
    model.load_state_dict(sd, strict=False, assign=True)
    for layer in model.layers:
        for blk, names in (("attention", ("wq", "wk", "wv", "wo")), ("feed_forward", ("w1", "w2", "w3"))):
            for name in names:
                lin = getattr(getattr(layer, blk), name)
                n_out, k_in = lin.shape
                v = (torch.randn((n_out, k_in), device=dev, generator=g) * 0.02).half()
                lin.w, lin.s = K.q_int40(v.t().contiguous(), 64)
                lin.shape = torch.Size((n_out, k_in))
    model.to(device=dev, dtype=torch.float16)
    model.eval()
    return model


def time_region(torch, fn, iters):
    """average milliseconds of fn() over `iters` calls, HIP events on the current stream"""
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    fn()
    torch.cuda.synchronize()
    start.record()
    for _ in range(iters):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / iters


def step_matmuls(model):
    """The weight-streaming launches of one decode step as the model issues them: per layer the fused
    wq|wk|wv, wo, the fused w1|w3 and w2 (128 launches for 32 layers)."""
    out = []
    for layer in model.layers:
        a, f = layer.attention, layer.feed_forward
        seg = lambda lin: (lin.operand(model.tiled_weights), lin.shape[0])      # (what the model hands the kernel, columns)
        out.append((a.wq.shape[1], [seg(a.wq), seg(a.wk), seg(a.wv)]))
        out.append((a.wo.shape[1], [seg(a.wo)]))
        out.append((f.w1.shape[1], [seg(f.w1), seg(f.w3)]))
        out.append((f.w2.shape[1], [seg(f.w2)]))
    return out


def matmul_roofline(torch, model, M, iters):
    """Only the Q4_0 matmul kernels (q40_gemv_kernel for M <= 16; above, the kernels the model launches at that batch:
    q40_gemm_kg_kernel, q40_gemm_swiglu_kernel for w1|w3 where it applies, q40_gemm_kernel otherwise), launched once per
    weight launch of a decode step at batch M, back to back in one HIP graph; timed with HIP events on the
    stream the graph runs on.  Every launch reads different weights (3.4 GB per pass, the Infinity Cache
    holds 256 MB)."""
    from spec_mcts_amd import kernels as K
    dev = torch.device("cuda:0")
    launches = step_matmuls(model)
    xs = {k: torch.randn((M, k), device=dev).half() for k in {k for k, _ in launches}}

    def run():
        for k_in, segs in launches:
            if len(segs) == 2 and model.swiglu_in_matmul and K.swiglu_fits(M, k_in, segs[0][1]):
                K.matmul_q40_swiglu(xs[k_in], segs[0][0], segs[1][0])       # w1|w3 as the model launches it at this batch
            else:
                K.matmul_q40_partial(xs[k_in], [op for op, _ in segs])

    run()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run()
    for _ in range(10):                  # clocks and caches settle before the timed replays
        graph.replay()
    ms = time_region(torch, graph.replay, iters)
    total_bytes = sum(sum(q40_bytes(0, n, k_in) for _, n in segs) + 2 * M * k_in + 4 * M * sum(n for _, n in segs)
                      for k_in, segs in launches)
    flops = sum(2 * M * k_in * sum(n for _, n in segs) for k_in, segs in launches)
    n = len(launches)
    return {"launches": n, "avg_us": ms * 1e3 / n, "bytes_per_launch": total_bytes / n, "gbs": total_bytes / (ms * 1e-3) / 1e9,
            "tflops": flops / (ms * 1e-3) / 1e12}


SWEEP_SHAPES = ((4096, 4096), (11008, 4096), (4096, 11008), (32128, 4096))     # (N, K); 32128 = vocab 32016 padded to 251 x 128 columns


def matmul_sweep(torch, iters=3):
    """BASELINE configs[1]: the Q4_0 matmul kernel alone at M = 1, 10, 100 on every CodeLlama-7B shape (the vocabulary
    projection zero-padded from 32016 to 32128 columns, the next multiple of 128 - the reference's format cannot hold 32016).
    Each point cycles through distinct weight copies that together exceed the 256 MB Infinity Cache, launched back to back
    in one HIP graph and timed with HIP events on its stream; weights in the tiled streaming layout, as the model holds
    them.  Bytes per launch: packed nibbles + scales + activations + fp16 outputs."""
    from spec_mcts_amd import kernels as K
    dev = torch.device("cuda:0")
    out = []
    for N, Kd in SWEEP_SHAPES:
        wbytes = N * Kd // 2 + N * Kd // 32
        copies = max(2, -(-300_000_000 // wbytes))
        tiled = []
        for _ in range(copies):
            w = torch.randint(-128, 128, (Kd * N // 128, 64), device=dev, dtype=torch.int16).to(torch.int8)
            s = (torch.rand((Kd * N // 64,), device=dev) * 0.01).half()
            tiled.append(K.tile_q40(w, s, Kd, N))
            del w, s
        for M in (1, 10, 100):
            x = torch.randn((M, Kd), device=dev).half()

            def run():
                for t in tiled:
                    K.matmul_q40_partial(x, [t])

            run()
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                run()
            for _ in range(3):
                graph.replay()
            us = time_region(torch, graph.replay, iters) * 1e3 / copies
            del graph
            # the same launch over ONE weight copy, repeated: the weights stay in the 256 MB Infinity Cache ("hot")
            hot = torch.cuda.CUDAGraph()
            with torch.cuda.graph(hot):
                for _ in range(8):
                    K.matmul_q40_partial(x, [tiled[0]])
            for _ in range(3):
                hot.replay()
            hot_us = time_region(torch, hot.replay, iters) * 1e3 / 8
            del hot
            nbytes = q40_bytes(M, N, Kd)
            flops = 2.0 * M * N * Kd
            out.append({"M": M, "N": N, "K": Kd, "us": round(us, 2), "bytes": nbytes, "gbs": round(nbytes / us / 1e3, 1),
                        "hbm_frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4), "tflops": round(flops / us / 1e6, 1),
                        "mfma_frac": round(flops / us / 1e6 / MFMA_F16_PEAK_TFLOPS, 4), "weight_copies": copies,
                        "hot_cache_us": round(hot_us, 2)})
        del tiled
        torch.cuda.empty_cache()
    return out


def attention_roofline(torch, iters=5, copies=3, fp16_suffix=False):
    """The shared-prefix decode attention alone on the reference's tree-attention shape: 64 branches, 32 heads,
    head_dim 128, one 1024-token fp16 prefix shared by all branches, ragged suffixes of 0..256 rows per branch held
    as the model stores them (Q4_0 rows + scales) or, with fp16_suffix, as fp16 rows (the shape as the reference's own
    check draws it), seed 2.  Algorithmic bytes: the prefix once, every valid suffix row once, q and out.  `copies`
    distinct caches alternate so that the suffix does not stay in the Infinity Cache."""
    from spec_mcts_amd import kernels as K
    dev = torch.device("cuda:0")
    B, H, D, P, S = 64, 32, 128, 1024, 256
    g = torch.Generator().manual_seed(2)
    lens = torch.randint(0, S + 1, (B,), generator=g, dtype=torch.int32)
    q = torch.randn((B, H, D), generator=g).half().to(dev)
    sets = []
    for _ in range(copies):
        pk, pv = torch.randn((P, H, D), device=dev).half(), torch.randn((P, H, D), device=dev).half()
        if fp16_suffix:
            sk, sv = torch.randn((B, S, H, D), device=dev).half(), torch.randn((B, S, H, D), device=dev).half()
            sks = svs = None
        else:
            sk = torch.randint(-128, 128, (B, S, H, 64), device=dev, dtype=torch.int16).to(torch.int8)
            sv = torch.randint(-128, 128, (B, S, H, 64), device=dev, dtype=torch.int16).to(torch.int8)
            sks, svs = (torch.rand((B, S, H, 2), device=dev) * 0.1).half(), (torch.rand((B, S, H, 2), device=dev) * 0.1).half()
        sets.append((pk, pv, sk, sv, sks, svs))
    lens_d = lens.to(dev)

    def run():
        for pk, pv, sk, sv, sks, svs in sets:
            K.shared_prefix_attn(q, pk, pv, P, suffix_k=sk, suffix_v=sv, suffix_ks=sks, suffix_vs=svs, Smax=S, lens=lens_d, lens_stride=1)

    run()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run()
    for _ in range(5):
        graph.replay()
    ms = time_region(torch, graph.replay, iters) / copies
    rows = int(lens.sum())
    nbytes = 2 * P * H * D * 2 + rows * H * 2 * (2 * D if fp16_suffix else 64 + 4) + 2 * B * H * D * 2
    return {"us": ms * 1e3, "bytes": nbytes, "gbs": nbytes / (ms * 1e-3) / 1e9, "suffix_rows": rows}


def tree_search_bench(torch, model, prompt, batch_sizes=(8, 16, 80, 100), depth=127, temp=0.8):
    """The reference's headline loop (load_q40.py:183-216): mcts(...).search(prompt, B) over batch sizes, tokens per second
    of the whole search (prefill included).  `tok_s` counts every token a live branch produced (the reference's "corrected"
    figure, sum of results_len), `tok_s_raw` rows x steps of the returned tensor (its raw figure).  Run with the decode
    steps replayed from per-bucket HIP graphs (the default) and issued launch by launch.  `expand_us` is the time of one
    expansion (sample_topk_counts + tree_step: draws, fork, terminal state machine, bookkeeping) at the full batch, HIP events
    over 20 calls."""
    from spec_mcts_amd import kernels as K
    from spec_mcts_amd.mcts import mcts, TERMINAL_SEQ, EOS
    dev = torch.device("cuda:0")
    out = []
    for B in batch_sizes:
        row = {"batch_size": B, "depth": depth, "top_k": 32, "temp": temp}
        for use_graph in (True, False):
            tree = mcts(model, depth, top_k=32, temp=temp)
            tree.use_graph = use_graph
            tree.generator = torch.Generator(device=dev).manual_seed(11)
            tree.search(prompt, B)                               # warm-up (captures the buckets' graphs)
            torch.cuda.synchronize()
            tree.generator.manual_seed(11)
            t0 = time.perf_counter()
            res, res_len, stats = tree.search(prompt, B)
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            key = "graph" if use_graph else "eager"
            row[key] = {"s": round(dt, 4), "tok_s": round(float(res_len.sum()) / dt, 1), "tok_s_raw": round(res.numel() / dt, 1),
                        "decode_steps": tree.last_steps, "graph_replays": tree.last_replays, "ms_per_step": round(dt / max(res.shape[1], 1) * 1e3, 3)}
            if use_graph:
                row["branches_at_end"] = int(res.shape[0])
                row["steps_to_full_batch"] = int((stats.cpu() < B).sum()) + 1
                row["host_reads_per_step"] = 1
        # one expansion step at the full batch, on logits of the right shape
        logits = torch.randn((B, model.vocab_size), device=dev).half()
        counts = torch.ones(B, dtype=torch.int32, device=dev)
        oc = torch.stack((torch.zeros_like(counts), counts)).contiguous()
        alive = torch.ones(B, dtype=torch.uint8, device=dev)
        curr_b = torch.full((1,), B, dtype=torch.int32, device=dev)
        results = torch.zeros((B, depth), dtype=torch.int64, device=dev)
        state = torch.zeros(B, dtype=torch.int32, device=dev)
        term = torch.tensor(TERMINAL_SEQ, dtype=torch.int64, device=dev)
        draws = torch.zeros(B, dtype=torch.int64, device=dev)
        u = torch.rand(B, device=dev)
        pages = model._table(dev).clone()
        t_dev = torch.full((1,), 5, dtype=torch.int32, device=dev)
        origin, res_len = torch.empty(B, dtype=torch.int32, device=dev), torch.zeros(B, dtype=torch.int32, device=dev)
        nxt, summary = torch.zeros(B, dtype=torch.int64, device=dev), torch.zeros(2, dtype=torch.int32, device=dev)

        def expand():
            K.sample_topk_counts(logits, temp, 32, oc[1], u, out=draws)
            K.tree_step(draws, oc, alive, curr_b, results, t_dev, pages, origin, state, term, res_len, nxt, summary, EOS)

        row["expand_us"] = round(time_region(torch, expand, 20) * 1e3, 2)
        out.append(row)
    return out


def paged_attention_bench(torch, iters=20):
    """The reference's tree-attention benchmark shape (triton_kernels_bench.py:495-552, stats/paged_flash_attn.csv): B branches
    over L = 512 positions, 32 heads of 128, a 256-page prompt shared by all, one fork per step until B branches exist, pools
    [H, P, D] fp16, int16 page ids; page_flash_attn alone, HIP events.  Algorithmic bytes: every DISTINCT page once (K and V),
    the page table, q and out."""
    from spec_mcts_amd import kernels as K
    dev = torch.device("cuda:0")
    L, H, D, prompt_L = 512, 32, 128, 256
    out = []
    for B in (64, 99):
        pager = torch.zeros((B, L), dtype=torch.int64)
        pager[:, :prompt_L] = torch.arange(prompt_L)
        page_idx, b = prompt_L, 1
        for i in range(prompt_L, L):
            if b < B:
                pager[b, :i] = pager[b - 1, :i]
                b += 1
            pager[:b, i] = page_idx + torch.arange(b)
            page_idx += b
        P = 1
        while P <= page_idx:
            P *= 2
        distinct = int(pager.unique().numel())
        pg = pager.to(torch.int16).to(dev)
        q = (torch.randn((B, H, D), device=dev) * 0.5).half()
        kp, vp = (torch.randn((H, P, D), device=dev) * 0.5).half(), (torch.randn((H, P, D), device=dev) * 0.5).half()
        fn = lambda: K.page_flash_attn(pg, q, kp, vp, P, B, L, H, D)
        fn()
        ms = time_region(torch, fn, iters)
        nbytes = 2 * distinct * H * D * 2 + B * L * 2 + 2 * B * H * D * 2
        out.append({"B": B, "L": L, "prompt": prompt_L, "ms": round(ms, 4), "distinct_pages": distinct, "bytes": nbytes,
                    "gbs": round(nbytes / (ms * 1e-3) / 1e9, 1), "hbm_frac": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)})
    return out


def cpu_baseline(torch, args_kw, prompt_len, budget_s=30.0):
    """The reference's CPU PyTorch path on ONE transformer layer (dequantise + F.linear for each of
    the 7 linears, explicit softmax attention over prompt + suffix), scaled by n_layers, plus the
    fp16 lm_head: the workload's prompt is prefilled, then decode steps are timed (median of up to 8 at 1 and
    10 branches, of up to 3 at 100).  Bounded to about `budget_s` seconds."""
    from oracle import q40_oracle as O
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    oargs = O.OracleArgs(**{**args_kw, "n_layers": 1, "max_batch_size": 100})
    sd = O.random_q40_state_dict(oargs, seed=7)
    model = O.OracleTransformer(oargs, sd, dense=False)     # dense=False: dequantise on every call, as the reference does
    P = prompt_len
    prompt = torch.randint(0, oargs.vocab_size, (1, P))
    t_start = time.perf_counter()
    model.forward(prompt, 0)
    t_prefill = time.perf_counter() - t_start
    res, n_steps = {}, {}
    for B in (1, 10, 100):
        tok = torch.randint(0, oargs.vocab_size, (B, 1))
        times = []
        for i in range(8 if B < 100 else 3):
            t0 = time.perf_counter()
            model.forward(tok, P + i)
            times.append(time.perf_counter() - t0)
            if time.perf_counter() - t_start > budget_s and len(times) >= 2:
                break
        res[B] = sorted(times)[len(times) // 2]
        n_steps[B] = len(times)
    # one forward() above = embedding + 1 layer + lm_head; time the head alone to scale layers only
    h = torch.randn((1, oargs.dim)).half()
    t0 = time.perf_counter()
    (h.float() @ sd["output.weight"].float().t()).half()
    t_head = time.perf_counter() - t0
    n_layers = args_kw["n_layers"]
    out = {}
    for B, t in res.items():
        step = max(t - t_head, 0.0) * n_layers + t_head
        out[B] = B / step
    return out, cores, {"steps": n_steps, "prefill_one_layer_s": round(t_prefill, 3)}


def single_linear_cpu_ms(torch):
    """The first configuration's case on the host: x [1, 4096] through one Q4_0 linear W [11008, 4096] with the reference's CPU
    recipe (dequantise the whole weight, then F.linear): median of 5 calls, milliseconds."""
    from oracle import q40_oracle as O
    g = torch.Generator().manual_seed(0)
    x = torch.randn((1, 4096), generator=g).half()
    v = (torch.randn((11008, 4096), generator=g) * 0.02).half()
    w, s, shape = O.quantize_weight(v)
    times = []
    for _ in range(5):
        t0 = time.perf_counter()
        O.linear_q40_cpu_path(x, w, s, shape)
        times.append(time.perf_counter() - t0)
    return round(sorted(times)[2] * 1e3, 3)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--no-norm-in-matmul", action="store_true", help="RMSNorm as its own launch at every batch size (comparison runs)")
    ap.add_argument("--norm-in-rows", type=int, default=-1, help="RMSNorm inside the matmul up to this many rows (comparison runs; default: the model's)")
    ap.add_argument("--batches", default="", help="comma-separated subset of 1,10,100 to run (a partial run is not a valid result)")
    ap.add_argument("--no-roofline", action="store_true", help="skip the matmul roofline legs (profiling runs)")
    ap.add_argument("--no-sweep", action="store_true", help="skip the per-shape matmul sweep, the eager-loop timing and the full-length decode")
    ap.add_argument("--no-tree", action="store_true", help="skip the tree-search and paged-attention legs")
    ap.add_argument("--roofline-only", type=int, default=0, metavar="M",
                    help="profiling aid: run only the matmul roofline leg at batch M (eager launches, one pass) after a 1 GiB "
                         "device copy that calibrates the profiler's byte counters, and print that leg's numbers")
    ap.add_argument("--attention-only", action="store_true",
                    help="profiling aid: run only the decode attention leg (64 branches, 1024-token shared prefix, ragged Q4_0 suffixes) "
                         "after the same 1 GiB calibration copy, and print that leg's numbers")
    ap.add_argument("--tree-only", action="store_true",
                    help="profiling aid: run only the tree-search leg (mcts.search, 512-token prompt, 8 .. 100 branches) and the paged "
                         "attention leg, and print their numbers")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers for a quick functional run (INVALID as a result)")
    ap.add_argument("--arch", choices=sorted(ARCHS), default="7b",
                    help="7b is the headline workload; 70b is the 80-layer GQA architecture with a 2048-token prompt (about 38 GB of Q4_0 "
                         "weights, run with --steps + --warmup < 64)")
    a = ap.parse_args()
    arch = dict(ARCHS[a.arch])
    prompt_len, max_seq = arch.pop("prompt"), arch.pop("max_seq_len")
    a.layers = a.layers or arch["n_layers"]
    if a.gpus != 1:
        sys.exit("bench.py: this build runs the Q4_0 decode path on ONE GPU; --gpus must be 1 "
                 "(branches would shard data-parallel across GPUs, which this run does not exercise)")
    import torch
    from spec_mcts_amd.decode import GraphDecoder

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    steps, warmup = a.steps, a.warmup
    assert steps + warmup + 1 <= max_seq, "this workload decodes at most %d tokens per branch" % max_seq
    args_kw = dict(arch, n_layers=a.layers, norm_eps=1e-5, rope_theta=1e6, max_batch_size=100, max_seq_len=max_seq,
                   max_prompt_seq_len=prompt_len)
    torch.manual_seed(3)
    model = build_model(torch, args_kw, seed=3)
    if a.no_norm_in_matmul:
        model.norm_in_matmul = False
    if a.norm_in_rows >= 0:
        model.norm_in_max_rows = a.norm_in_rows
    prompt = torch.randint(0, 32016, (1, prompt_len), generator=torch.Generator().manual_seed(3)).cuda()

    if a.roofline_only or a.attention_only:
        src = torch.empty(1 << 29, dtype=torch.float16, device="cuda:0").normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)                                     # 1 GiB read + 1 GiB written by one elementwise kernel
        torch.cuda.synchronize()
        del src, dst
        print(json.dumps(attention_roofline(torch) if a.attention_only else matmul_roofline(torch, model, a.roofline_only, 3)))
        return
    if a.tree_only:
        print(json.dumps({"tree_search": tree_search_bench(torch, model, prompt), "paged_attn": paged_attention_bench(torch)}))
        return
    batches = tuple(int(x) for x in a.batches.split(",")) if a.batches else BATCHES
    # the prefill of the shared prompt (once per tree, outside the timed decode steps): reported next to them
    dec = GraphDecoder(model, 1, use_graph=False)
    dec.prefill(prompt)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    dec.prefill(prompt)
    torch.cuda.synchronize()
    prefill_ms = (time.perf_counter() - t0) * 1e3
    del dec
    by_batch = {}
    for B in batches:
        dec = GraphDecoder(model, B, use_graph=not a.no_graph)
        dec.prefill(prompt)
        dec.capture()
        dec.decode(warmup)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        dec.decode(steps)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        by_batch[B] = {"tok_s": B * steps / dt, "ms_per_step": dt / steps * 1e3}
        if not a.no_sweep:
            # the workload as the configuration words it: every decode step the suffix cache holds after the prefill's
            # token (max_seq_len - 1 steps), whatever --steps says, timed as one run of the captured graph
            full = max_seq - 1
            dec.prefill(prompt)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            dec.decode(full)
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            by_batch[B]["decode_full"] = {"steps": full, "tok_s": B * full / dt, "ms_per_step": dt / full * 1e3}
        del dec
        if not a.no_sweep:
            # the same steps issued launch by launch from Python, as mcts.search's model(tokens, pos) calls would issue them
            dec = GraphDecoder(model, B, use_graph=False)
            dec.prefill(prompt)
            dec.decode(warmup)                              # the same suffix positions as the graph's timed steps
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            dec.decode(steps)
            torch.cuda.synchronize()
            by_batch[B]["eager_ms_per_step"] = (time.perf_counter() - t0) / steps * 1e3
            del dec

    # per-step algorithmic HBM bytes: Q4 linears + fp16 lm_head + shared prefix KV (once) + suffix KV (Q4 rows)
    lin_bytes = sum(q40_bytes(0, n, k_in) for k_in, segs in step_matmuls(model) for _, n in segs)
    kv_heads = model.layers[0].attention.n_kv_heads
    kv_dim = kv_heads * 128
    head_bytes = 32016 * arch["dim"] * 2
    prefix_bytes = 2 * prompt_len * kv_dim * 2 * a.layers
    suffix_row_bytes = a.layers * 2 * kv_heads * 68          # K and V, 64 nibble bytes + 2 fp16 scales per head
    t_mid = warmup + steps // 2
    for B in batches:
        step_bytes = lin_bytes + head_bytes + prefix_bytes + B * t_mid * suffix_row_bytes
        by_batch[B]["hbm_frac"] = step_bytes / (by_batch[B]["ms_per_step"] * 1e-3) / 1e9 / HBM_PEAK_GBS

    head = by_batch.get(100) or by_batch[max(by_batch)]
    head_b = 100 if 100 in by_batch else max(by_batch)
    result = {
        "metric": "Q4_0 %s decode tok/s at B=1/10/100; Q4_0 GEMV achieved HBM GB/s" % a.arch.upper(),
        "value": head["tok_s"], "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "codellama%s_arch_q40_decode_prompt%d_shared_prefix" % (a.arch, prompt_len), "branches": head_b,
                   "layers": a.layers, "graph": not a.no_graph},
        "by_batch": {str(B): {k: (round(v, 4) if isinstance(v, float) else ({kk: round(vv, 4) for kk, vv in v.items()} if isinstance(v, dict) else v))
                              for k, v in d.items()} for B, d in by_batch.items()},
        "prefill": {"prompt_tokens": prompt_len, "ms": round(prefill_ms, 3), "tok_s": round(prompt_len / (prefill_ms * 1e-3), 1)},
    }
    if not a.no_roofline:
        rf1 = matmul_roofline(torch, model, 1, 5)
        rf10 = matmul_roofline(torch, model, 10, 5)
        rf100 = matmul_roofline(torch, model, 100, 3)
        result["roofline"] = {
            "kernel": "q40_gemv_kernel at M=1: the %d weight launches of one %s decode step (wq|wk|wv, wo, w1|w3, w2 per layer)"
                      % (rf1["launches"], a.arch.upper()),
            "bound": "hbm", "achieved": round(rf1["gbs"], 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(rf1["gbs"] / HBM_PEAK_GBS, 4), "traffic": GEMV_TRAFFIC_BYTES_PER_LAUNCH if a.arch == "7b" else None,
            "avg_launch_us": round(rf1["avg_us"], 3), "bytes_per_launch": round(rf1["bytes_per_launch"])}
        result["rooflines_other"] = [
            {"kernel": "q40_gemv_kernel at M=10", "bound": "hbm", "achieved": round(rf10["gbs"], 1), "peak": HBM_PEAK_GBS,
             "unit": "GB/s", "frac": round(rf10["gbs"] / HBM_PEAK_GBS, 4), "avg_launch_us": round(rf10["avg_us"], 3)},
            {"kernel": "Q4_0 GEMM at M=100: q40_gemm_kg_kernel (wq|wk|wv, wo, w2) and q40_gemm_swiglu_kernel (w1|w3), the 128 weight launches of a step", "bound": "mfma", "achieved": round(rf100["tflops"], 1),
             "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(rf100["tflops"] / MFMA_F16_PEAK_TFLOPS, 4),
             "hbm_gbs": round(rf100["gbs"], 1), "avg_launch_us": round(rf100["avg_us"], 3), "traffic": GEMM_TRAFFIC_BYTES_PER_LAUNCH if a.arch == "7b" else None},
        ]
        att = attention_roofline(torch)
        result["rooflines_other"].append(
            {"kernel": "attn_prefix_kernel + attn_suffix_kernel: 64 branches x 32 heads, shared 1024-token fp16 prefix, ragged Q4_0 "
                       "suffixes of 0..256 rows (the two launches of one call)",
             "bound": "hbm", "achieved": round(att["gbs"], 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
             "frac": round(att["gbs"] / HBM_PEAK_GBS, 4), "avg_call_us": round(att["us"], 2), "bytes_per_call": att["bytes"], "traffic": ATTN_TRAFFIC_BYTES_PER_CALL})
        att16 = attention_roofline(torch, fp16_suffix=True)
        result["rooflines_other"].append(
            {"kernel": "attn_prefix_kernel + attn_suffix_kernel: the same shape with the suffixes as fp16 rows (512 B per row and head "
                       "instead of 136 B)",
             "bound": "hbm", "achieved": round(att16["gbs"], 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
             "frac": round(att16["gbs"] / HBM_PEAK_GBS, 4), "avg_call_us": round(att16["us"], 2), "bytes_per_call": att16["bytes"], "traffic": None})
    if not a.no_sweep and a.arch == "7b":
        result["matmul_sweep"] = matmul_sweep(torch)
    if not a.no_tree and a.arch == "7b" and a.layers == arch["n_layers"]:
        result["tree_search"] = tree_search_bench(torch, model, prompt)
        result["paged_attn"] = paged_attention_bench(torch)
    if not a.no_cpu_baseline:
        cpu, cores, raw = cpu_baseline(torch, args_kw, prompt_len)
        result["cpu_baseline"] = {"value": round(cpu.get(head_b, cpu.get(max(cpu), 0.0)), 4), "unit": "tok/s", "cores": cores, "kind": "port",
                                  "sample": "oracle CPU path (torch dequantise + F.linear, fp32 compute): one layer + lm_head after a "
                                            "%d-token prefill, median of %s decode steps at B=1, 10, 100, layer time x n_layers; "
                                            "value is the B=%d figure" % (prompt_len, "/".join(str(raw["steps"][B]) for B in sorted(raw["steps"])), head_b),
                                  "prefill_one_layer_s": raw["prefill_one_layer_s"],
                                  "by_batch": {str(B): round(v, 4) for B, v in cpu.items()},
                                  "single_linear_ms": single_linear_cpu_ms(torch)}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
