"""Tree sampler of the reference (mcts.py: class mcts, search) on the device operators of this package.

Same constructor and call: mcts(model, depth, nodes, top_k, temp).search(prompt, batch_size) returns
(results[:curr_batch], results_len, batch_stats) as mcts.py:67-182 does.  What differs is where the work runs: the
expansion step - counts[i] draws per branch, torch.unique, one new row per further distinct token, Transformer.fork per
branch in a Python loop with a host round trip per tensor element (mcts.py:127-152) - is two launches
(kernels.sample_topk_counts, kernels.tree_fork), a fork is a copy of page ids inside the second of them, and the host
reads back two integers per step in one copy (the number of live branches, which sizes the next forward, and the
number of ended rows, which stops the search).

Randomness: the draws are inverse-CDF draws over uniform numbers from torch.rand (the generator may be passed in) in place
of torch.multinomial's stream, so token sequences differ from the reference's for the same seed while the distribution
of every draw is the same.  The decode steps run as captured HIP graphs, one per batch-size bucket (decode.BucketedForward;
`use_graph = False` issues the same launches one by one): the batch grows between steps, and at a few branches a step is
bound by how fast the host can issue its ~260 launches.  temp > 0: one temperature for all branches; temp <= 0: the reference's ramp, branch i at
0.1 + (|temp| - 0.1) (n_i - 1) / (batch_size - 1) for multiplicity n_i (mcts.py:110-114), in float32 as there.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import kernels as K

TERMINAL_SEQ = (29961, 29914, 20055, 4690, 1164, 29962)       # "[/PYTHON]" (mcts.py:12)
EOS = 2


class mcts:
    def __init__(self, model, depth, nodes: int = 1024 ** 2, top_k: int = 32, temp: float = 0.3):
        self.max_nodes = nodes
        self.top_k = top_k
        self.max_depth = depth
        self.max_batch = model.params.max_batch_size
        self.model = model
        self.temp = temp
        self.generator: Optional[torch.Generator] = None
        self.verbose = False
        self.use_graph = True
        self._fwd = None
        self.last_steps = 0           # decode steps of the last search, and how many of them replayed a graph
        self.last_replays = 0
        self.last_counts = None

    @torch.inference_mode()
    def search(self, prompt: torch.Tensor, batch_size: int):
        """Grow up to batch_size branches from one prompt until every live branch has ended or max_depth tokens exist."""
        m = self.model
        assert m.paged_kv, "the device-side fork copies page ids: paged_kv must be on"
        m.resetTimers()
        m.resetSeq()
        assert m.params.max_batch_size >= batch_size
        dev = m.norm.weight.device
        idx = prompt[:1].to(dev)
        assert m.params.max_prompt_seq_len >= idx.shape[1]
        steps = min(self.max_depth, m.params.max_seq_len)
        results = torch.zeros((batch_size, steps), dtype=torch.int64, device=dev)
        results_len = torch.zeros(batch_size, dtype=torch.int32, device=dev)
        alive = torch.ones(batch_size, dtype=torch.bool, device=dev)                 # results_mask
        output_counts = torch.zeros((2, batch_size), dtype=torch.int32, device=dev)
        output_counts[1, 0] = batch_size
        curr_b = torch.ones(1, dtype=torch.int32, device=dev)
        curr = 1
        batch_stats = torch.zeros(steps, dtype=torch.uint8, device=dev)
        state = torch.zeros(batch_size, dtype=torch.int32, device=dev)               # end_stateMachine
        terminal = torch.tensor(TERMINAL_SEQ, dtype=torch.int64, device=dev)
        draws = torch.zeros(batch_size, dtype=torch.int64, device=dev)
        origin = torch.empty(batch_size, dtype=torch.int32, device=dev)
        fwd = None
        if m.fused and not m.per_branch_kv:
            from .decode import BucketedForward
            if self._fwd is None or self._fwd.model is not m or self._fwd.max_batch != batch_size or self._fwd.use_graph != self.use_graph:
                self._fwd = BucketedForward(m, batch_size, use_graph=self.use_graph)
            fwd = self._fwd
        replays0 = fwd.replays if fwd is not None else 0
        pos = 0
        for t in range(steps):
            if pos == 0:
                logits = m(idx, 0)
                pos = idx.shape[1]
                if fwd is not None:
                    fwd.begin()
            elif fwd is not None:
                logits = fwd.step(results[:curr, t - 1:t])
                pos += 1
            else:
                logits = m(results[:curr, t - 1:t], pos)
                pos += 1
            logits = logits[:, -1, :]
            u = torch.rand(batch_size, device=dev, dtype=torch.float32, generator=self.generator)
            if self.temp > 0.0:
                temperature = self.temp
            else:       # mcts.py:113-114, the expression itself: int32 tensor -> float32 (ZeroDivisionError at batch_size 1, as there)
                temperature = ((abs(self.temp) - 0.1) / (batch_size - 1) * (output_counts[1] - 1) + 0.1).contiguous()
            K.sample_topk_counts(logits, temperature, self.top_k, output_counts[1], u, out=draws)
            # the new rows read their ancestors' suffix rows through the model's page table: rows 0 .. t-1 exist so far
            K.tree_fork(draws, output_counts, alive, curr_b, results, t, pages=m._table(dev), n_rows=m._rows_written, origin=origin)
            ends, state = K.detect_terminal(results[:, t].contiguous(), state, terminal, EOS)
            results_len += alive.int()
            alive = ~(ends | ~alive)
            new_curr, ended = torch.stack((curr_b[0], (~alive).sum().int())).tolist()     # the step's one host read
            if new_curr > curr and m._rows_written > 0:
                m._forked = True
            curr = new_curr
            batch_stats[t] = curr
            if self.verbose:
                print(f"step {t}: {curr} branches, {int(alive[:curr].sum())} alive")
            if ended == curr:                                                        # mcts.py:174 (counts ended rows over the whole batch)
                steps = t + 1
                break
        self.last_steps = steps - 1
        self.last_counts = output_counts      # (token, multiplicity) per row after the last step (mcts.py:154-155's invariant)
        self.last_replays = fwd.replays - replays0 if fwd is not None else 0
        m.printTimers()
        return results[:curr, :steps], results_len, batch_stats[:steps]
