"""The Python entry point: model folder (or configuration + seed) to generated tokens.

    engine = LLMEngine("path/to/model")                    # or LLMEngine(config=cfg, seed=0)
    outs = engine.generate([[1, 2, 3], [4, 5]], SamplingParams(max_tokens=16))

``generate`` runs the scheduler loop: admit, cut prompts into portions under the
token budget, decode, sample on the GPU, finish and free. ``add_request`` /
``step`` / ``abort`` expose the same loop one step at a time, ``step_raw`` is the
step function itself (what trace replay drives). The reference's single-request
loop is bin/reinfer/src/pipeline.rs:123-239 and its batching loop
bin/reinfer/src/sched_loop.rs:691-1029; it re-runs the last prompt token as the
first decode step (pipeline.rs:173-178), here the first token is sampled from
the logits at the prompt's last position.
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Union

import torch

from ..config import load_config
from ..sampling import Sampler, SamplingError, SamplingParams, derive_seed
from .batch import StepEntry
from .runner import ModelRunner
from .scheduler import FINISHED, Request, RequestRefused, Scheduler, StepPlan


@dataclass
class RequestOutput:
    rid: Hashable
    prompt_token_ids: List[int]
    token_ids: List[int]
    finish_reason: Optional[str]
    preemptions: int = 0


class LLMEngine:
    def __init__(self, model: Optional[str] = None, *, config=None, seed: int = 0,
                 dtype: str = "bfloat16", device: str = "cuda:0", weights=None,
                 max_model_len: Optional[int] = None, block_size: int = 16,
                 num_blocks: Optional[int] = None, max_num_seqs: int = 64,
                 max_num_batched_tokens: int = 2048, max_chunk: Optional[int] = None,
                 memory_fraction: float = 0.9, admission: str = "peak", allow_unexpected: bool = False):
        limits = dict(block_size=block_size, num_blocks=num_blocks, max_seqs=max_num_seqs,
                      max_model_len=max_model_len, memory_fraction=memory_fraction)
        if model is not None:
            self.config = load_config(model)
            self.runner = ModelRunner.from_folder(model, dtype=dtype, device=device,
                                                  allow_unexpected=allow_unexpected, **limits)
        elif config is not None:
            self.config = config
            self.runner = ModelRunner.from_config(config, seed=seed, dtype=dtype, device=device,
                                                  weights=weights, **limits)
        else:
            raise ValueError("give a model folder, or a configuration (random weights from the seed)")
        self.seed = int(seed)
        self.device = self.runner.device
        self.scheduler = Scheduler(self.runner.manager, max_num_seqs=max_num_seqs,
                                   max_num_batched_tokens=max_num_batched_tokens,
                                   max_model_len=self.runner.max_model_len, max_chunk=max_chunk,
                                   eos_token_ids=self.runner.spec.eos_token_ids, admission=admission)
        self.sampler = Sampler(self.device)
        self._pending = None        # the step launched last: (plan, requests that sample, device tokens, host tokens, event)
        pin = self.device.type == "cuda"
        self._token_buffers = [torch.zeros(max(1, int(max_num_seqs)), dtype=torch.int32, pin_memory=pin) for _ in range(2)]
        self._token_turn = 0
        self._auto_id = 0
        self.timings: Dict[str, float] = {}

    # --------------------------------------------------------- requests
    def add_request(self, prompt_token_ids: Sequence[int], params: Optional[SamplingParams] = None,
                    rid: Optional[Hashable] = None) -> Hashable:
        params = params or SamplingParams()
        if rid is None:
            rid = f"req-{self._auto_id}"
            self._auto_id += 1
        V = self.runner.spec.vocab_size
        for t in prompt_token_ids:
            if not 0 <= int(t) < V:
                raise RequestRefused(f"token {t} outside the vocabulary of {V}")
        arrival = self.scheduler.num_arrivals
        seed = params.seed if params.seed is not None else derive_seed(self.seed, arrival)
        self.scheduler.add(rid, [int(t) for t in prompt_token_ids], params, seed)
        return rid

    def abort(self, rid: Hashable) -> bool:
        return self.scheduler.abort(rid)

    def has_unfinished(self) -> bool:
        return self.scheduler.has_work() or self._pending is not None

    # -------------------------------------------------------------- step
    # A step is launched in one call and its tokens are read in the next: between the two the scheduler
    # has advanced every request by the place of its token (``advance_blind``) and plans the step after it
    # without the token's value. Where that next step is the same requests decoding again, it is launched
    # at once, its tokens handed over on the device (the captured step's input buffer is filled from the
    # sampler's output buffer), and only then are the earlier step's tokens read: the GPU goes from one
    # decode step to the next without waiting for the host. A request that a token ended (an end-of-sequence
    # or stop id) has by then one more row in flight; the row is dropped (``resolve``). What the scheduler
    # assumes: whether a request goes on after a step does not depend on the step's token, until it is told
    # otherwise one step later; so a request ended by a token leaves one step later than it might, and a
    # waiting request takes its place one step later. Tokens do not depend on any of this: a request's
    # noise is a function of its seed and position.
    def step(self) -> List[RequestOutput]:
        """One scheduler decision and one batch launched; the tokens of the batch launched by the call
        before are read, and the requests they ended are returned."""
        pending = self._pending
        plan = self.scheduler.schedule()
        finished = [self._output(r) for r in plan.finished]
        if pending is None:
            if not plan.portions:
                if not finished and self.scheduler.has_work() and not plan.preempted:
                    raise RuntimeError("the scheduler could place no token although work is waiting")
                return finished
            self._launch(plan, None)
            return finished
        if plan.portions and self._chains(pending, plan):
            self._launch(plan, pending)
            done = self._resolve(pending)
        else:
            # the next step needs tokens the host has to see first (a prompt's first token, a row that a
            # filter shapes), or is another set of rows: read, then launch
            done = self._resolve(pending)
            self._pending = None
            if plan.portions:
                self._launch(plan, None)
            elif not finished and not done and self.scheduler.has_work() and not plan.preempted:
                raise RuntimeError("the scheduler could place no token although work is waiting")
        return finished + [self._output(r) for r in done]

    def _chains(self, pending, plan: StepPlan) -> bool:
        """The planned step is the one just launched over again: the same requests, one token each, all
        drawn inside the captured step."""
        return pending[2] is not None and self.runner.can_chain(len(pending[1])) \
            and self.scheduler.repeats(pending[0], plan)

    def _launch(self, plan: StepPlan, chained_from) -> None:
        # a request that an earlier token ended since the plan was made has no part in the step
        entries, rows, sampling = self.scheduler.entries_for(plan)
        if not entries:
            self._pending = None
            return
        if chained_from is not None:
            logits, toks = self.runner.step_sampled(entries, sampling, token_source=chained_from[2][:len(rows)])
        else:
            logits, toks = self.runner.step_sampled(entries, sampling)
        tokens_host = event = None
        if toks is not None:
            # out of the step's own buffer (the next replay overwrites it) into pinned memory, without waiting
            tokens_host = self._token_buffers[self._token_turn][:len(rows)]
            self._token_turn ^= 1
            tokens_host.copy_(toks, non_blocking=True)
            event = torch.cuda.Event()
            event.record()
        elif rows:
            tokens_host = self.sampler.sample(logits, [r.params for r in rows], [r.seed for r in rows],
                                              [r.num_tokens for r in rows], [r.tokens for r in rows])
        else:
            tokens_host = []
        self.scheduler.advance_blind(plan)
        self._pending = (plan, rows, toks, tokens_host, event)

    def _resolve(self, pending) -> List[Request]:
        plan, rows, _, tokens_host, event = pending
        if event is not None:
            event.synchronize()
            out = tokens_host.tolist()
            if out and min(out) < 0:
                r = rows[[t < 0 for t in out].index(True)]
                raise SamplingError(f"request {r.rid!r}: no finite logit to sample from")
        else:
            out = list(tokens_host)
        return self.scheduler.resolve(plan, out)

    @staticmethod
    def _output(r: Request) -> RequestOutput:
        return RequestOutput(r.rid, list(r.prompt), list(r.output), r.finish_reason, r.preemptions)

    def step_raw(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """The step function itself: given tokens in, float32 logits out, no sampling."""
        return self.runner.step(entries)

    # ---------------------------------------------------------- generate
    def generate(self, prompt_token_ids: Sequence[Sequence[int]],
                 sampling_params: Union[SamplingParams, Sequence[SamplingParams], None] = None
                 ) -> List[RequestOutput]:
        if isinstance(sampling_params, SamplingParams) or sampling_params is None:
            sampling_params = [sampling_params or SamplingParams()] * len(prompt_token_ids)
        if len(sampling_params) != len(prompt_token_ids):
            raise ValueError("one SamplingParams per prompt")
        rids = [self.add_request(p, sp) for p, sp in zip(prompt_token_ids, sampling_params)]
        outs: Dict[Hashable, RequestOutput] = {}
        t0 = time.perf_counter()
        first = None
        while self.has_unfinished():
            for o in self.step():
                outs[o.rid] = o
            if first is None:
                first = time.perf_counter() - t0
        self.timings = {"total_s": time.perf_counter() - t0, "first_step_s": first or 0.0}
        return [outs[r] for r in rids]

    def get_weight(self, name: str) -> torch.Tensor:
        """The tensor ``name`` as the model was given it, on the CPU (see ModelRunner.get_weight)."""
        return self.runner.get_weight(name)

    def cache_stats(self) -> Dict[str, object]:
        s = self.runner.manager.stats()
        s.update(self.scheduler.counters)
        return s
