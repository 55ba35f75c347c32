"""Greedy tree-branch decoding with the whole decode step captured in one HIP graph.

A decode step of the 7B model is ~420 kernel launches of a few microseconds each; issued one by
one from Python the step is launch-bound.  The kernels read the position and the suffix index
from device memory, so one captured graph serves every step: replay, bump the two counters on the
device, replay again.  No hipMemsetAsync node is recorded (the matmul workspace cleans itself).
"""
from __future__ import annotations

from typing import Optional

import torch

from . import kernels as K
from .hf_model_q40_kv_shared import Transformer


class GraphDecoder:
    """Prefill once at B=1, share the prompt KV between `batch_size` branches, then greedy-decode.

    Equivalent to calling model(tokens, start_pos) + argmax step by step (the graph records exactly
    those kernels); `use_graph=False` runs that eager loop instead.
    """

    def __init__(self, model: Transformer, batch_size: int, use_graph: bool = True):
        assert batch_size <= model.params.max_batch_size
        self.model = model
        self.B = batch_size
        self.use_graph = use_graph
        self.device = model.norm.weight.device
        self.tokens = torch.zeros((batch_size, 1), dtype=torch.int64, device=self.device)
        self.state = torch.zeros(2, dtype=torch.int32, device=self.device)     # (position, suffix index)
        self.one = torch.ones(2, dtype=torch.int32, device=self.device)
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self._graph_key = None        # what the captured launches were planned for: (prompt length, model switches)
        self._pinned = []             # workspaces whose addresses are inside the graph: kept alive as long as it is
        self.prompt_len = 0
        self.t = 0                    # suffix rows written so far (host mirror of state[1])

    def _step(self):
        logits = self.model._forward_impl(self.tokens, 1, (self.state[0:1], self.state[1:2]))
        K.argmax(logits.view(self.B, -1), out=self.tokens)      # the next step's input, written in place
        self.state.add_(self.one)

    @torch.inference_mode()
    def prefill(self, prompt: torch.Tensor) -> torch.Tensor:
        """prompt int64 [1,P] -> first greedy token; resets the branch state."""
        m = self.model
        m.resetSeq()
        logits = m(prompt[:1].to(self.device), 0)[:, -1]
        self.prompt_len = m.layers[0].attention.cache_prompt_len      # (a prompt longer than the cache was cropped by the model)
        first = K.argmax(logits.contiguous())
        self.tokens.copy_(first.view(1, 1).expand(self.B, 1))
        self._reset_state()
        if self.graph is not None and self._graph_key != self._key():
            # the prompt length decides the attention's slices, grid and workspace layout, all constants of the
            # recorded launches: a graph captured for another prompt length is dropped and captured again
            self.graph = None
        return first

    def _key(self):
        m = self.model
        return (self.prompt_len, self.B, m.fused, m.tiled_weights, m.silu_in_matmul, m.swiglu_in_matmul, m.norm_in_matmul, m.norm_in_max_rows,
                m.attn_from_qkv, m.attn_single_launch, m.per_branch_kv, m._forked)

    def _reset_state(self):
        self.state.copy_(torch.tensor([self.prompt_len, 0], dtype=torch.int32))
        self.t = 0

    @torch.inference_mode()
    def capture(self):
        """Warm up (allocates workspaces, loads kernels) and record one decode step."""
        saved = self.tokens.clone()
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            for _ in range(2):
                self._reset_state()
                self._step()
        torch.cuda.current_stream().wait_stream(s)
        torch.cuda.synchronize()
        self._reset_state()
        self.tokens.copy_(saved)
        if self.use_graph:
            # the warm-up grew the shared workspaces to what this step needs; the graph records their addresses, so
            # they must outlive it even if a later, larger call replaces them in the operators' table
            self._pinned = list(K._workspaces.values())
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph):
                self._step()
            self._graph_key = self._key()
            # the capture pass itself does not execute; state and tokens are untouched
        torch.cuda.synchronize()

    @torch.inference_mode()
    def decode(self, steps: int, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Run `steps` decode steps; returns the tokens produced, int64 [B, steps]."""
        if out is None:
            out = torch.empty((self.B, steps), dtype=torch.int64, device=self.device)
        p = self.model.params
        # the kernels take position and suffix row from device counters and do not know the caches' ends
        assert self.t + steps <= p.max_seq_len, f"suffix cache exhausted: {self.t} + {steps} rows of {p.max_seq_len}"
        assert self.prompt_len + self.t + steps <= self.model.freqs_cis.shape[0], "position beyond the rotation table"
        assert self.graph is None or self._graph_key == self._key(), "the graph was captured for another prompt length or configuration"
        self.t += steps
        self.model._rows_written = self.t
        for i in range(steps):
            if self.graph is not None:
                self.graph.replay()
            else:
                self._step()
            out[:, i].copy_(self.tokens[:, 0])
        return out

    @torch.inference_mode()
    def generate(self, prompt: torch.Tensor, steps: int) -> torch.Tensor:
        """tokens [B, steps]: the first comes from the prefill logits, the rest from decode steps."""
        first = self.prefill(prompt)
        if self.graph is None and self.use_graph:
            self.capture()
        res = torch.empty((self.B, steps), dtype=torch.int64, device=self.device)
        res[:, 0] = first
        if steps > 1:
            self.decode(steps - 1, res[:, 1:])
        return res


class BucketedForward:
    """Decode-step forward for a batch that grows between steps (the tree sampler: mcts.py:96-102 calls
    model(results[:curr_batch_size, t-1:t], pos) with more rows after every fork).

    One HIP graph per batch-size bucket (1, 2, 4, ... and the largest batch): a step with `curr` live branches replays the
    graph of the smallest bucket that holds them.  The rows past `curr` are computed too; they read the token buffer's stale
    entries and append K/V to their own cache rows at the step's suffix index - rows no page table refers to, because a
    branch that is created later reads its ancestors' positions through the page ids copied at the fork and writes its own
    from the fork's step on.  Position and suffix index live on the device and are advanced by the graph itself, so the
    same graph serves every step; graphs are captured when a bucket is first needed and kept while the prompt length and
    the model's switches stay the same.  The page table is always in use (identity until the first fork), so that the fork
    does not change what the recorded launches read.  `post(logits)` - set by the caller, None for none - is issued right
    behind the forward and recorded with it (the tree sampler's draws and bookkeeping: they take the step index from
    `state[1]` and leave the next step's tokens in `tokens`), so a whole search step is one replay.
    """

    def __init__(self, model: Transformer, max_batch: int, use_graph: bool = True):
        assert max_batch <= model.params.max_batch_size
        self.model = model
        self.max_batch = max_batch
        self.use_graph = use_graph
        self.device = model.norm.weight.device
        b, self.buckets = 1, []
        while b < max_batch:
            self.buckets.append(b)
            b *= 2
        self.buckets.append(max_batch)
        self.tokens = torch.zeros((max_batch, 1), dtype=torch.int64, device=self.device)
        self.state = torch.zeros(2, dtype=torch.int32, device=self.device)     # (position, suffix index)
        self.one = torch.ones(2, dtype=torch.int32, device=self.device)
        self.graphs = {}              # bucket -> (graph, logits [bucket, 1, vocab])
        self._key = None
        self._pinned = []
        self.prompt_len = 0
        self.t = 0
        self.replays = 0
        self.post = None
        self.post_key = None

    def _config(self):
        m = self.model
        return (self.prompt_len, m.fused, m.tiled_weights, m.silu_in_matmul, m.swiglu_in_matmul, m.norm_in_matmul, m.norm_in_max_rows, m.attn_from_qkv,
                m.attn_single_launch, m.per_branch_kv)

    def begin(self):
        """After the prefill: take the prompt length from the model, rewind the suffix, switch the page table on."""
        m = self.model
        assert m.paged_kv and not m.per_branch_kv, "the growing batch shares suffix rows through the page table"
        self.prompt_len = m.layers[0].attention.cache_prompt_len
        self.state.copy_(torch.tensor([self.prompt_len, 0], dtype=torch.int32))
        self.t = 0
        m._forked = True
        if self._key != self._config():
            self.graphs = {}
            self._key = self._config()

    def _run(self, bucket: int):
        logits = self.model._forward_impl(self.tokens[:bucket], 1, (self.state[0:1], self.state[1:2]))
        self.state.add_(self.one)
        if self.post is not None:
            self.post(logits)
        return logits

    def bucket_of(self, curr: int) -> int:
        return next(b for b in self.buckets if b >= curr)

    @torch.inference_mode()
    def step(self, tokens: Optional[torch.Tensor], curr: int = 0) -> torch.Tensor:
        """tokens int64 [curr, 1] (the previous step's tokens of the live branches; None: `curr` rows of the token buffer
        are already in place) -> logits fp16 [curr, 1, vocab]"""
        curr = tokens.shape[0] if tokens is not None else curr
        p = self.model.params
        assert 1 <= curr <= self.max_batch
        assert self.t < p.max_seq_len, "suffix cache exhausted"
        assert self.prompt_len + self.t < self.model.freqs_cis.shape[0], "position beyond the rotation table"
        bucket = self.bucket_of(curr)
        if tokens is not None:
            self.tokens[:curr].copy_(tokens)
        if not self.use_graph:
            logits = self._run(bucket)
        else:
            if bucket not in self.graphs:
                self._capture(bucket)
            graph, logits = self.graphs[bucket]
            graph.replay()
            self.replays += 1
        self.t += 1
        self.model._rows_written = self.t
        return logits[:curr]

    def _capture(self, bucket: int):
        saved = self.state.clone()
        post, self.post = self.post, None         # the warm-up runs the forward only: `post` changes the caller's state
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            for _ in range(2):                    # warm-up at the current step: what it appends the replay writes again
                self.state.copy_(saved)
                self._run(bucket)
        torch.cuda.current_stream().wait_stream(s)
        torch.cuda.synchronize()
        self.state.copy_(saved)
        self.post = post
        # the warm-up grew the shared workspaces to what this bucket needs; the graph records their addresses
        self._pinned.extend(w for w in K._workspaces.values() if not any(w is q for q in self._pinned))
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            logits = self._run(bucket)
        self.graphs[bucket] = (g, logits)
        torch.cuda.synchronize()
