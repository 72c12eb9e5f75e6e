"""Decode steps as captured HIP graphs.

A step in which every request brings exactly one token has the same shape each
time; only index arrays change. Such a step is captured once per (padded batch
size, context bucket) with static input buffers, and later steps copy their
indices into those buffers (one host-to-device copy) and replay the graph: the
few hundred launches of a step cost one call. The captured work is the
product's own forward pass and sampler, run through the same parts and kernels
as an eager step; nothing is traced or rewritten.

Rows past the step's requests are padding: token 0 at position 0 that stores
nothing (slot -1, state slot -1) and whose logits nobody reads. A part that keeps
per-request state and declares itself ``graph_safe`` must leave state slot -1
alone.

The reference launches every kernel of every step from the host
(crates/cuda/src/engine.rs:5853-6350) and names graph capture as future work.
"""
from __future__ import annotations

import gc
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from .. import kernels
from .._hostlib import host as host_runtime
from .batch import StepBatch, StepEntry

MAX_GRAPH_BATCH = 128


def _bucket(n: int) -> int:
    b = 1
    while b < n:
        b *= 2
    return b


def _batch_bucket(n: int) -> int:
    """Rows a captured step is padded to: powers of two up to 32, from there multiples of 16 (the
    products work in tiles of 16 rows: from 17 rows on a product's time grows with the number of its
    row tiles, and so would the padding's cost; 33 requests padded to 48 rows instead of 64:
    7.5 -> 7.0 ms a step at the Qwen3-8B shape)."""
    return _bucket(n) if n <= 32 else -(-n // 16) * 16


class _CapturedStep:
    """Static buffers and the graph of one (batch size, context bucket)."""

    def __init__(self, runner, B: int, ctx_cap: int, pool):
        self.runner = runner
        self.B = B
        self.ctx_cap = ctx_cap
        dev = runner.device
        bs = runner.block_size
        n_groups = len(runner.manager.groups)
        W = max(1, -(-runner.max_model_len // bs))
        self.W = W
        # layout of the packed int32 buffer (seeds first: they are read as int64)
        names = [("seeds", 2 * B), ("temps", B), ("sample_pos", B), ("token_ids", B), ("positions", B),
                 ("seq_of_token", B), ("cu_tokens", B + 1), ("start_pos", B), ("ctx_lens", B),
                 ("state_slots", B), ("fresh", B), ("logit_rows", B), ("no_slots", B)]
        for g in range(n_groups):
            names += [(f"table{g}", B * W), (f"slots{g}", B)]
        self.off: Dict[str, Tuple[int, int]] = {}
        o = 0
        for name, size in names:
            self.off[name] = (o, o + size)
            o += size
        self.host = torch.zeros(o, dtype=torch.int32, pin_memory=True)
        self.h = self.host.numpy()
        self.dev = torch.zeros(o, dtype=torch.int32, device=dev)

        def hv(name):
            a, b = self.off[name]
            return self.h[a:b]

        def dv(name):
            a, b = self.off[name]
            return self.dev[a:b]

        # what never changes
        hv("seq_of_token")[:] = np.arange(B)
        hv("cu_tokens")[:] = np.arange(B + 1)
        hv("logit_rows")[:] = np.arange(B)
        hv("no_slots")[:] = -1
        # the host runtime keeps track of which request sits in which row and writes what changed
        order = ["token_ids", "positions", "start_pos", "ctx_lens", "state_slots", "fresh", "sample_pos",
                 "temps", "seeds"]
        for g in range(n_groups):
            order += [f"table{g}", f"slots{g}"]
        self.rows = host_runtime.DecodeRows(runner.manager, B, W, [self.off[k][0] for k in order])
        self.rows.pad_all(self.h)

        self.seeds = dv("seeds").view(torch.int64)
        self.temps = dv("temps").view(torch.float32)
        self.sample_pos = dv("sample_pos")
        self.tokens = torch.zeros(B, dtype=torch.int32, device=dev)
        self.batch = StepBatch(
            num_tokens=B, num_seqs=B, num_logit_rows=B,
            token_ids=dv("token_ids"), positions=dv("positions"), seq_of_token=dv("seq_of_token"),
            cu_tokens=dv("cu_tokens"), start_pos=dv("start_pos"), ctx_lens=dv("ctx_lens"),
            state_slots=dv("state_slots"), fresh=dv("fresh"), logit_rows=dv("logit_rows"),
            no_slots=dv("no_slots"),
            block_tables=[dv(f"table{g}").view(B, W) for g in range(n_groups)],
            slots=[dv(f"slots{g}") for g in range(n_groups)],
            q_lens=[1] * B, starts=[ctx_cap - 1] * B, max_q_len=1, max_ctx_len=ctx_cap)
        # the kernels choose grids from host-side numbers: the parts fix them for this bucket
        runner.model.plan_captured_step(self.batch, B, ctx_cap)
        self.logits: Optional[torch.Tensor] = None
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.copied: Optional[torch.cuda.Event] = None      # behind the last copy out of the staging buffer
        self._capture(pool)

    def _body(self) -> None:
        r = self.runner
        self.logits = r.model.forward(self.batch, r.caches)
        kernels.current().sample(self.logits, self.temps, self.seeds, self.sample_pos, self.tokens)

    def _capture(self, pool) -> None:
        self.dev.copy_(self.host, non_blocking=True)
        # once outside the capture: whatever initialises lazily must not be recorded
        cur = torch.cuda.current_stream()
        side = torch.cuda.Stream()
        side.wait_stream(cur)
        with torch.cuda.stream(side), torch.no_grad():
            self._body()
        cur.wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        # No garbage collection inside the capture: a dead cycle that holds device memory or a graph
        # of its own (an earlier runner with its captured steps) would be destroyed in the middle of
        # it, and releasing device memory while a stream captures is an error that ends the process.
        # Such cycles are collected here, before the capture begins.
        gc.collect()
        was_enabled = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(self.graph, pool=pool), torch.no_grad():
                self._body()
        finally:
            if was_enabled:
                gc.enable()

    def fill(self, entries: List[StepEntry], sampling) -> None:
        # The staging buffer is the source of the last replay's copy, which the GPU may not have made
        # yet if nobody read that step's results (a step with no logits wanted): wait for that copy
        # before the buffer is written again, or the last step would run with this step's indices.
        if self.copied is not None:
            self.copied.synchronize()
        self.rows.fill(entries, self.h, sampling)

    def replay(self, token_source: Optional[torch.Tensor] = None) -> None:
        self.dev.copy_(self.host, non_blocking=True)
        if self.copied is None:
            self.copied = torch.cuda.Event()
        self.copied.record()
        if token_source is not None:
            # the step's tokens are those that the step before it drew, still on the device: they take the
            # place of what the host wrote (it does not know them yet)
            n = token_source.numel()
            self.batch.token_ids[:n].copy_(token_source, non_blocking=True)
        self.graph.replay()


class DecodeGraphs:
    def __init__(self, runner):
        self.runner = runner
        self.steps: Dict[Tuple[int, int], _CapturedStep] = {}
        self.pool = None
        self.replays = 0

    def run(self, entries: List[StepEntry], longest: int, sampling=None, token_source: Optional[torch.Tensor] = None):
        """A step of at most MAX_GRAPH_BATCH entries with one token each; ``longest`` is the longest
        context after it. -> (logits [B_pad, vocab] static, tokens [B_pad] static): rows past the
        entries are padding; both are overwritten by the next replay of this bucket. ``token_source``: an
        int32 device tensor, one token per entry, that replaces the entries' own tokens (the tokens of the
        step before, which the host has not read yet)."""
        r = self.runner
        B = _batch_bucket(len(entries))
        # context buckets are powers of two from 256, and never more than the block tables hold (a
        # context limit that is no power of two, or below 256, is its own last bucket)
        table_room = max(1, -(-r.max_model_len // r.block_size)) * r.block_size
        ctx_cap = min(max(256, _bucket(longest)), table_room)
        key = (B, ctx_cap)
        cs = self.steps.get(key)
        if cs is None:
            if self.pool is None:
                self.pool = torch.cuda.graph_pool_handle()
            cs = _CapturedStep(r, B, ctx_cap, self.pool)
            self.steps[key] = cs
        cs.fill(entries, sampling)
        cs.replay(token_source)
        self.replays += 1
        return cs.logits, cs.tokens
