"""Tree sampler of the reference (mcts.py: class mcts, search) on the device operators of this package.

Same constructor and call: mcts(model, depth, nodes, top_k, temp).search(prompt, batch_size) returns
(results[:curr_batch], results_len, batch_stats) as mcts.py:67-182 does.  What differs is where the work runs: the
expansion step - counts[i] draws per branch, torch.unique, one new row per further distinct token, Transformer.fork per
branch in a Python loop with a host round trip per tensor element (mcts.py:127-152) - is two launches
(kernels.sample_topk_counts, kernels.tree_step), a fork is a copy of page ids inside the second of them, which also runs
the terminal state machine and the row bookkeeping of mcts.py:160-175; and the host reads back two integers per step in
one copy (the number of live branches, which sizes the next forward, and the number of ended rows, which stops the search).
With the fused forward a whole search step - the decode step, the draws, the bookkeeping - is ONE replay of a captured HIP
graph per batch-size bucket (decode.BucketedForward; `use_graph = False` issues the same launches one by one): the batch
grows between steps, and at a few branches a step is bound by how fast the host can issue its ~260 launches.

Randomness: the draws are inverse-CDF draws over uniform numbers from torch.rand (the generator may be passed in) in place
of torch.multinomial's stream, so token sequences differ from the reference's for the same seed while the distribution
of every draw is the same.  temp > 0: one temperature for all branches; temp <= 0: the reference's ramp, branch i at
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
        self._buf = None
        self._pinned = None
        self.last_issued = 0          # decode steps issued (one more than last_steps when the end was seen a step late)

    @torch.inference_mode()
    def search(self, prompt: torch.Tensor, batch_size: int):
        """Grow up to batch_size branches from one prompt until every live branch has ended or max_depth tokens exist."""
        m = self.model
        assert m.paged_kv, "the device-side fork copies page ids: paged_kv must be on"
        assert m.params.max_batch_size >= batch_size
        if m.fused and not m.per_branch_kv:
            return self._search_fused(prompt, batch_size)
        return self._search_stepwise(prompt, batch_size)

    # -- the fused path: a search step = one graph replay (forward + draws + the whole bookkeeping) and one host read --------
    def _buffers(self, batch_size: int, steps: int, dev):
        key = (batch_size, steps, str(dev))
        if self._buf is None or self._buf["key"] != key:
            i32 = dict(dtype=torch.int32, device=dev)
            self._buf = dict(
                key=key,
                results=torch.zeros((batch_size, steps), dtype=torch.int64, device=dev),
                results_len=torch.zeros(batch_size, **i32),
                alive=torch.ones(batch_size, dtype=torch.uint8, device=dev),              # results_mask
                output_counts=torch.zeros((2, batch_size), **i32),
                curr_b=torch.ones(1, **i32),
                state=torch.zeros(batch_size, **i32),                                     # end_stateMachine
                terminal=torch.tensor(TERMINAL_SEQ, dtype=torch.int64, device=dev),
                draws=torch.zeros(batch_size, dtype=torch.int64, device=dev),
                origin=torch.empty(batch_size, **i32),
                u=torch.zeros(batch_size, dtype=torch.float32, device=dev),
                summary=torch.zeros(2, **i32))
        return self._buf

    def _search_fused(self, prompt: torch.Tensor, batch_size: int):
        from .decode import BucketedForward
        m = self.model
        m.resetTimers()
        m.resetSeq()
        dev = m.norm.weight.device
        idx = prompt[:1].to(dev)
        assert m.params.max_prompt_seq_len >= idx.shape[1]
        steps = min(self.max_depth, m.params.max_seq_len)
        b = self._buffers(batch_size, steps, dev)
        b["results"].zero_(); b["results_len"].zero_(); b["alive"].fill_(1); b["output_counts"].zero_(); b["state"].zero_()
        b["output_counts"][1, 0] = batch_size
        b["curr_b"].fill_(1)
        if (self._fwd is None or self._fwd.model is not m or self._fwd.max_batch != batch_size or self._fwd.use_graph != self.use_graph
                or self._fwd.post_key != (id(b), self.temp, self.top_k)):
            self._fwd = BucketedForward(m, batch_size, use_graph=self.use_graph)
            self._fwd.post_key = (id(b), self.temp, self.top_k)       # what the recorded draws and bookkeeping were given
        fwd = self._fwd
        temp, top_k = self.temp, self.top_k

        def expand(logits):
            """draws + the step's bookkeeping on logits [rows, vocab]; every argument lives at a fixed address"""
            if temp > 0.0:
                temperature = temp
            else:       # mcts.py:113-114, the expression itself: int32 tensor -> float32 (ZeroDivisionError at batch_size 1, as there)
                temperature = ((abs(temp) - 0.1) / (batch_size - 1) * (b["output_counts"][1] - 1) + 0.1).contiguous()
            K.sample_topk_counts(logits, temperature, top_k, b["output_counts"][1], b["u"], out=b["draws"])
            # the new rows read their ancestors' suffix rows through the model's page table: rows 0 .. t-1 exist so far
            K.tree_step(b["draws"], b["output_counts"], b["alive"], b["curr_b"], b["results"], fwd.state[1:2], m._table(dev), b["origin"],
                        b["state"], b["terminal"], b["results_len"], fwd.tokens.view(-1), b["summary"], EOS)

        fwd.post = lambda logits: expand(logits[:, -1, :])
        replays0 = fwd.replays
        # The host reads (branches, ended rows) once per step.  While the batch can still outgrow its bucket the read comes
        # before the next step is issued; once the largest bucket is in use the next step's graph is fixed, so it is issued
        # FIRST and the numbers of the step before are read while it runs (from pinned memory, behind an event): the GPU does
        # not wait for the host between steps.  The end of the search is then seen one step late; that step runs on rows
        # that have all ended (it adds nothing to their lengths and writes zeros) and its column is cut off.
        if self._pinned is None:
            self._pinned = (torch.zeros((2, 2), dtype=torch.int32).pin_memory(), [torch.cuda.Event(), torch.cuda.Event()])
        host, events = self._pinned
        curr, stats = 1, []
        issued = 0                       # steps whose launches are enqueued
        done = False
        while not done:
            if issued < steps and (issued == len(stats) or fwd.bucket_of(curr) == fwd.buckets[-1]):
                t = issued
                b["u"].copy_(torch.rand(batch_size, device=dev, dtype=torch.float32, generator=self.generator))
                if t == 0:
                    logits = m(idx, 0)
                    fwd.begin()
                    expand(logits[:, -1, :])
                else:
                    fwd.step(None, curr)                             # tokens: left in place by the previous step
                host[t & 1].copy_(b["summary"], non_blocking=True)
                events[t & 1].record()
                issued += 1
                if issued - len(stats) < 2 and issued < steps and t > 0 and fwd.bucket_of(curr) == fwd.buckets[-1]:
                    continue                                         # one step ahead of the host's reads
            t = len(stats)
            events[t & 1].synchronize()
            curr, ended = host[t & 1].tolist()                       # the step's one host read
            stats.append(curr)
            if self.verbose:
                print(f"step {t}: {curr} branches, {ended} rows ended")
            if ended == curr or len(stats) == steps:                 # mcts.py:174 (counts ended rows over the whole batch)
                steps = len(stats)
                done = True
        torch.cuda.synchronize()                                     # (a step issued ahead may still run)
        if issued > steps:
            # rows that no branch ever took count as live in the reference's bookkeeping (results_len += results_mask, :163):
            # the steps that ran past the end lengthened them
            b["results_len"][curr:] -= issued - steps
        self.last_steps = steps - 1
        self.last_issued = issued - 1
        self.last_replays = fwd.replays - replays0
        self.last_counts = b["output_counts"].clone()
        m.printTimers()
        return b["results"][:curr, :steps].clone(), b["results_len"].clone(), torch.tensor(stats, dtype=torch.uint8, device=dev)

    # -- the step-by-step path (module-by-module forward, or every position in the branch's own cache) -------------------------
    def _search_stepwise(self, prompt: torch.Tensor, batch_size: int):
        m = self.model
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
        pos = 0
        for t in range(steps):
            if pos == 0:
                logits = m(idx, 0)
                pos = idx.shape[1]
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
        self.last_replays = 0
        m.printTimers()
        return results[:curr, :steps], results_len, batch_stats[:steps]
