"""Continuous batching above the step function (host logic only). The classes
are the C++ host runtime's (reinfer_amd/csrc/host/host.cpp); this module names them.

Each call of :meth:`Scheduler.schedule` decides one step: every decoding request
takes one token first; what is left of the token budget goes to prompt portions,
requests already running before waiting ones, resumed ones before new arrivals,
then first come first served (crates/scheduler/src/batch.rs:69-101,
policy.rs:30-63). A portion may be cut anywhere; it need not end on a block's
edge (the reference aligns to pages because it copies pages,
bin/reinfer/src/sched_loop.rs:1158-1163).

Admission (``admission="peak"``, the default): a waiting request joins the running ones only
while the estimated peak of what the set will hold fits the pool. Every request has a pair
(a, b): a = the tokens it holds once its current tokens are cached, b = the new tokens it is
expected to add yet (its cap when more than 0.8 of the pool is taken, else up to the larger of
1.1 x what it has generated and a running mean of finished requests' output lengths, plus 16);
with the set sorted by b descending the peak is max_k (b_k (k + 1) + a_0 + ... + a_k)
(crates/scheduler/src/admission.rs:72-86, 138-148, 211-240). A lone request always runs.
``admission="blocks"`` lets a request in as soon as the blocks of its first portion are free.

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

from .._hostlib import RequestRefused, host

WAITING, RUNNING, FINISHED = host.WAITING, host.RUNNING, host.FINISHED

# Request: rid, prompt, params, seed, arrival, state, output, num_computed (tokens of prompt +
#   output whose keys are in the cache), resumed, finish_reason, preemptions; tokens, num_tokens,
#   remaining, decoding (in the cache up to its last token, which is a generated one);
#   token_at(i), tokens_slice(start, n) read without copying the whole sequence.
# Portion: request, start, length; samples = the portion reaches the request's current end.
# StepPlan: portions, preempted, finished (ended without running: cache), num_tokens.
# Scheduler(manager, *, max_num_seqs, max_num_batched_tokens, max_model_len, max_chunk=None,
#           eos_token_ids=(), admission="peak"): add, abort, has_work, schedule, complete, pool_tokens; waiting,
#   running, requests, counters, budget.
Request = host.Request
Portion = host.Portion
StepPlan = host.StepPlan
Scheduler = host.Scheduler

__all__ = ["WAITING", "RUNNING", "FINISHED", "RequestRefused", "Request", "Portion", "StepPlan", "Scheduler"]
