"""Continuous batching above the step function (host logic only).

Each call of :meth:`Scheduler.schedule` decides one step: every decoding request
takes one token first; what is left of the token budget goes to prompt portions,
requests already running before waiting ones, resumed ones before new arrivals,
then first come first served (crates/scheduler/src/batch.rs:69-101,
policy.rs:30-63). A portion may be cut anywhere; it need not end on a block's
edge (the reference aligns to pages because it copies pages,
bin/reinfer/src/sched_loop.rs:1158-1163).

When blocks run out: before a step, if giving every decoding request its next
token needs more blocks than are free, the newest arrival among the running
requests is preempted (requests preempted before go last, policy.rs:59-63): all
its blocks are given back and it returns to the head of the waiting queue. On
resume it is recomputed from its prompt plus the tokens it had generated
(crates/scheduler/src/req.rs:340-357 recomputes from scratch), so its output is
what it would have been. A lone request that cannot get another block ends with
reason "cache". A prompt that could never fit is refused at submit.

Everything is a pure function of the arrival order: two runs decide the same
(crates/scheduler/src/replay.rs:1-7).
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, Hashable, List, Optional, Sequence, Tuple

from ..cache import CacheManager
from ..sampling.params import SamplingParams

WAITING, RUNNING, FINISHED = "waiting", "running", "finished"


class RequestRefused(ValueError):
    pass


@dataclass
class Request:
    rid: Hashable
    prompt: List[int]
    params: SamplingParams
    seed: int
    arrival: int
    state: str = WAITING
    output: List[int] = field(default_factory=list)
    num_computed: int = 0           # tokens of prompt + output whose keys are in the cache
    resumed: bool = False           # preempted at least once
    finish_reason: Optional[str] = None
    preemptions: int = 0

    @property
    def tokens(self) -> List[int]:
        return self.prompt + self.output

    @property
    def num_tokens(self) -> int:
        return len(self.prompt) + len(self.output)

    @property
    def remaining(self) -> int:
        return self.num_tokens - self.num_computed

    @property
    def decoding(self) -> bool:
        """In the cache up to its last token, which is a generated one."""
        return self.state == RUNNING and len(self.output) > 0 and self.remaining == 1


@dataclass
class Portion:
    request: Request
    start: int
    length: int

    @property
    def samples(self) -> bool:
        """The portion reaches the request's current end: its last logits give a token."""
        return self.start + self.length == self.request.num_tokens


@dataclass
class StepPlan:
    portions: List[Portion] = field(default_factory=list)
    preempted: List[Request] = field(default_factory=list)
    finished: List[Request] = field(default_factory=list)     # ended without running (cache)

    @property
    def num_tokens(self) -> int:
        return sum(p.length for p in self.portions)


class Scheduler:
    def __init__(self, manager: CacheManager, *, max_num_seqs: int, max_num_batched_tokens: int,
                 max_model_len: int, max_chunk: Optional[int] = None,
                 eos_token_ids: Sequence[int] = ()):
        if max_num_seqs < 1 or max_num_batched_tokens < 1:
            raise ValueError("max_num_seqs and max_num_batched_tokens must be positive")
        self.manager = manager
        self.max_num_seqs = min(max_num_seqs, manager.slots.num_slots)
        self.budget = max_num_batched_tokens
        self.max_model_len = max_model_len
        self.max_chunk = max_chunk or max_num_batched_tokens
        self.eos = set(int(t) for t in eos_token_ids)
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []
        self.requests: Dict[Hashable, Request] = {}
        self._arrivals = 0
        self.counters = {"steps": 0, "preemptions": 0, "finished": 0, "refused": 0, "tokens": 0}

    # ------------------------------------------------------------- intake
    def pool_tokens(self) -> int:
        return min(p.num_blocks for p in self.manager.pools) * self.manager.block_size

    def add(self, rid: Hashable, prompt: Sequence[int], params: SamplingParams, seed: int) -> Request:
        if rid in self.requests and self.requests[rid].state != FINISHED:
            raise RequestRefused(f"request {rid!r} is already live")
        if len(prompt) == 0:
            self.counters["refused"] += 1
            raise RequestRefused("empty prompt")
        if len(prompt) + 1 > self.max_model_len:
            self.counters["refused"] += 1
            raise RequestRefused(f"prompt of {len(prompt)} tokens leaves no room in a context of {self.max_model_len}")
        if len(prompt) + 1 > self.pool_tokens():
            self.counters["refused"] += 1
            raise RequestRefused(f"prompt of {len(prompt)} tokens can never fit a cache of {self.pool_tokens()} tokens")
        req = Request(rid=rid, prompt=list(int(t) for t in prompt), params=params, seed=seed,
                      arrival=self._arrivals)
        self._arrivals += 1
        self.requests[rid] = req
        self.waiting.append(req)
        return req

    def abort(self, rid: Hashable) -> bool:
        """Idempotent; frees once (crates/scheduler/src/req.rs:326-338)."""
        req = self.requests.get(rid)
        if req is None or req.state == FINISHED:
            return False
        if req.state == RUNNING:
            self.running.remove(req)
            self.manager.free(rid)
        else:
            self.waiting.remove(req)
        req.state, req.finish_reason = FINISHED, "abort"
        return True

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ------------------------------------------------------------ a step
    def _free_blocks(self) -> List[int]:
        return [p.num_free for p in self.manager.pools]

    def _held(self, req: Request) -> List[int]:
        rc = self.manager.get(req.rid)
        return [sum(1 for b in t if b >= 0) for t in rc.tables]

    def _preempt(self, req: Request, plan: StepPlan) -> None:
        self.running.remove(req)
        self.manager.free(req.rid)
        req.state, req.num_computed, req.resumed = WAITING, 0, True
        req.preemptions += 1
        self.counters["preemptions"] += 1
        self.waiting.appendleft(req)
        plan.preempted.append(req)

    def schedule(self) -> StepPlan:
        plan = StepPlan()
        n_groups = len(self.manager.groups)
        budget = self.budget

        # 1. decoding requests: one token each; make room by preempting the newest
        while True:
            decoders = [r for r in self.running if r.decoding]
            need = [0] * n_groups
            for r in decoders:
                for g, n in enumerate(self.manager.blocks_needed(r.rid, r.num_computed + 1)):
                    need[g] += n
            free = self._free_blocks()
            short = any(need[g] > free[g] for g in range(n_groups)) or len(decoders) > budget
            if not short:
                break
            # victims: not yet preempted first, newest arrival first (policy.rs:59-63)
            victims = sorted(self.running, key=lambda r: (r.resumed, -r.arrival))
            if len(self.running) == 1:
                lone = self.running[0]
                self.running.remove(lone)
                self.manager.free(lone.rid)
                lone.state, lone.finish_reason = FINISHED, "cache"
                self.counters["finished"] += 1
                plan.finished.append(lone)
                break
            self._preempt(victims[0], plan)
        decoders = sorted((r for r in self.running if r.decoding), key=lambda r: r.arrival)
        free = self._free_blocks()
        for r in decoders:
            for g, n in enumerate(self.manager.blocks_needed(r.rid, r.num_computed + 1)):
                free[g] -= n
            plan.portions.append(Portion(r, r.num_computed, 1))
            budget -= 1

        # 2. prompt portions of running requests, oldest first
        def fit(req: Request, start: int, want: int, live: bool, reserve: int = 0) -> int:
            """Largest portion <= want whose blocks are free (leaving ``reserve``
            blocks in every group); takes them from ``free``."""
            bs = self.manager.block_size
            n = want
            while n > 0:
                if live:
                    need = self.manager.blocks_needed(req.rid, start + n)
                else:
                    need = [-(-(start + n) // bs)] * n_groups
                if all(need[g] + reserve <= free[g] for g in range(n_groups)):
                    for g in range(n_groups):
                        free[g] -= need[g]
                    return n
                # shrink to the last block edge that fits
                n = min(n - 1, ((start + n - 1) // bs) * bs - start)
            return 0

        for r in sorted((r for r in self.running if not r.decoding), key=lambda r: r.arrival):
            if budget <= 0:
                break
            n = fit(r, r.num_computed, min(r.remaining, self.max_chunk, budget), True)
            if n > 0:
                plan.portions.append(Portion(r, r.num_computed, n))
                budget -= n

        # 3. admissions: resumed first (they sit at the head), then arrival order
        while self.waiting and budget > 0 and len(self.running) < self.max_num_seqs:
            r = self.waiting[0]
            if any(p is r for p in plan.preempted):
                break                   # preempted in this very step: not before the next
            # a block of headroom for every running request, so that an admission
            # does not force a preemption at the very next step
            n = fit(r, 0, min(r.remaining, self.max_chunk, budget), False, reserve=len(self.running))
            if n == 0:
                break                   # first come first served: nobody overtakes
            self.waiting.popleft()
            self.manager.add(r.rid)
            r.state = RUNNING
            self.running.append(r)
            plan.portions.append(Portion(r, 0, n))
            budget -= n

        # requests keep their order in the batch: by arrival (batch.rs:13-15 sorts by id)
        plan.portions.sort(key=lambda p: p.request.arrival)
        self.counters["steps"] += 1
        self.counters["tokens"] += plan.num_tokens
        return plan

    # ------------------------------------------------------ after a step
    def complete(self, plan: StepPlan, sampled: Dict[Hashable, int]) -> List[Request]:
        """The step ran: advance cursors, append sampled tokens, finish and free.

        Order of the checks: stop ids, then the cap on new tokens, then the
        context (crates/scheduler/src/req.rs:281-314: stop, EOS, max output);
        the stop token is consumed, not emitted.
        """
        done: List[Request] = []
        for p in plan.portions:
            r = p.request
            r.num_computed = p.start + p.length
            if not p.samples:
                continue
            tok = int(sampled[r.rid])
            stop = (tok in self.eos and not r.params.ignore_eos) or tok in r.params.stop_token_ids
            if stop:
                r.finish_reason = "stop"
            else:
                r.output.append(tok)
                if len(r.output) >= r.params.max_tokens:
                    r.finish_reason = "length"
                elif r.num_tokens >= self.max_model_len:
                    r.finish_reason = "length"
            if r.finish_reason is not None:
                r.state = FINISHED
                self.running.remove(r)
                self.manager.free(r.rid)
                self.counters["finished"] += 1
                done.append(r)
        return done
