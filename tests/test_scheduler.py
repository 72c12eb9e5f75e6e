"""The scheduler's decisions, without a model: a fake step whose sampled token is a
pure function of (request, position), as the reference's MockExecutor does
(bin/reinfer/src/sched_loop.rs:1594-1776)."""
import pytest

import plain_qwen3 as plain
from reinfer_amd.cache import CacheGroupSpec, CacheManager
from reinfer_amd.engine.scheduler import FINISHED, RUNNING, WAITING, RequestRefused, Scheduler
from reinfer_amd.sampling import SamplingParams


def make(num_blocks=64, bs=4, max_seqs=8, budget=32, max_model_len=512, max_chunk=None, eos=(), windows=(0,),
         admission="blocks"):
    groups = [CacheGroupSpec(window=w, entries=(i,)) for i, w in enumerate(windows)]
    m = CacheManager(groups, bs, [num_blocks] * len(groups), max_seqs)
    s = Scheduler(m, max_num_seqs=max_seqs, max_num_batched_tokens=budget, max_model_len=max_model_len,
                  max_chunk=max_chunk, eos_token_ids=eos, admission=admission)
    return m, s


def fake_token(rid, position, vocab=1000):
    return plain.splitmix64(hash(str(rid)) % (1 << 32) * 7919 + position) % vocab


def run_step(m, s, log=None, token_fn=fake_token):
    plan = s.schedule()
    assert plan.num_tokens <= s.budget
    for p in plan.portions:
        assert p.start == p.request.num_computed, "a portion starts where the cache ends"
        m.grow(p.request.rid, p.start + p.length)
    for p in plan.portions:
        m.commit(p.request.rid, p.start + p.length)
    sampled = {p.request.rid: token_fn(p.request.rid, p.request.num_tokens) for p in plan.portions if p.samples}
    if log is not None:
        log.append(([(p.request.rid, p.start, p.length) for p in plan.portions],
                    [r.rid for r in plan.preempted]))
    done = s.complete(plan, sampled)
    m.check()
    return plan, done


def drive(m, s, log=None, limit=10000, token_fn=fake_token):
    outs = {}
    n = 0
    while s.has_work():
        plan, done = run_step(m, s, log, token_fn)
        for r in done + plan.finished:
            outs[r.rid] = (list(r.output), r.finish_reason)
        n += 1
        assert n < limit, "the scheduler does not terminate"
    return outs


def test_decode_first_then_portion_under_budget():
    """batch.rs:128-142 with an effective budget of 8: three decoders take 3, the
    prompt of 40 gets [0, 5)."""
    m, s = make(budget=8, max_chunk=16)
    for i in range(3):
        s.add(f"d{i}", [1, 2], SamplingParams(max_tokens=50), seed=i)
    run_step(m, s)                              # prompts of 2 tokens each: 6 tokens
    assert all(r.decoding for r in s.running)
    s.add("p", list(range(40)), SamplingParams(max_tokens=5), seed=9)
    plan, _ = run_step(m, s)
    got = [(p.request.rid, p.start, p.length) for p in plan.portions]
    assert got == [("d0", 2, 1), ("d1", 2, 1), ("d2", 2, 1), ("p", 0, 5)]
    # continuation starts at the computed length (batch.rs:174-179)
    plan, _ = run_step(m, s)
    assert ("p", 5, 5) in [(p.request.rid, p.start, p.length) for p in plan.portions]


def test_max_chunk_and_fcfs():
    m, s = make(budget=64, max_chunk=16)
    s.add("a", list(range(40)), SamplingParams(max_tokens=2), seed=0)
    s.add("b", list(range(10)), SamplingParams(max_tokens=2), seed=0)
    plan, _ = run_step(m, s)
    assert [(p.request.rid, p.start, p.length) for p in plan.portions] == [("a", 0, 16), ("b", 0, 10)]
    plan, _ = run_step(m, s)        # b decodes, a continues
    assert [(p.request.rid, p.start, p.length) for p in plan.portions] == [("a", 16, 16), ("b", 10, 1)]


def test_exactly_max_tokens_and_stop_ids():
    m, s = make()
    s.add("a", [5, 6, 7], SamplingParams(max_tokens=7), seed=0)
    outs = drive(m, s)
    assert len(outs["a"][0]) == 7 and outs["a"][1] == "length"
    # an end-of-sequence id is consumed, not emitted (req.rs:281-314)
    m, s = make(eos=(42,))
    s.add("a", [1], SamplingParams(max_tokens=20), seed=0)
    seq = iter([3, 4, 42, 5])
    outs = drive(m, s, token_fn=lambda rid, pos: next(seq))
    assert outs["a"] == ([3, 4], "stop")
    m, s = make(eos=(42,))
    s.add("a", [1], SamplingParams(max_tokens=4, ignore_eos=True, stop_token_ids=(5,)), seed=0)
    seq = iter([3, 42, 5, 6])
    assert drive(m, s, token_fn=lambda rid, pos: next(seq))["a"] == ([3, 42], "stop")


def test_context_limit_ends_a_request():
    m, s = make(max_model_len=10)
    s.add("a", [1] * 6, SamplingParams(max_tokens=100), seed=0)
    outs = drive(m, s)
    assert len(outs["a"][0]) == 4 and outs["a"][1] == "length"      # 6 + 4 = 10 tokens
    with pytest.raises(RequestRefused, match="context"):
        s.add("b", [1] * 10, SamplingParams(), seed=0)


def test_refusals():
    m, s = make(num_blocks=4, bs=4)             # 16 tokens of cache
    with pytest.raises(RequestRefused, match="empty"):
        s.add("a", [], SamplingParams(), seed=0)
    with pytest.raises(RequestRefused, match="never fit"):
        s.add("a", [1] * 16, SamplingParams(), seed=0)
    s.add("a", [1] * 15, SamplingParams(max_tokens=1), seed=0)
    with pytest.raises(RequestRefused, match="already live"):
        s.add("a", [1], SamplingParams(), seed=0)
    assert s.counters["refused"] == 2


def test_preemption_newest_first_and_same_output():
    """Pages run out while decoding: the newest arrival is preempted, goes to the
    head of the queue, is recomputed, and ends with the output it would have had."""
    def run(num_blocks):
        m, s = make(num_blocks=num_blocks, bs=4, budget=64, max_seqs=4)
        for i, n in enumerate([9, 7, 8]):
            s.add(f"r{i}", list(range(1, n + 1)), SamplingParams(max_tokens=30), seed=i)
        log = []
        outs = drive(m, s, log)
        assert all(p.num_free == p.num_blocks for p in m.pools)
        return outs, log, s
    big, _, s_big = run(64)
    small, log, s_small = run(16)               # 64 tokens of cache for 3 x ~39
    assert s_big.counters["preemptions"] == 0 and s_small.counters["preemptions"] > 0
    assert small == big
    first = next(pre for _, pre in log if pre)
    assert first[0] == "r2", "the newest arrival goes first (policy.rs:59-63)"
    # a resumed request restarts at position 0 with prompt + generated tokens
    step_after = next(i for i, (_, pre) in enumerate(log) if pre)
    resumed = [x for portions, _ in log[step_after + 1:] for x in portions if x[0] == "r2"][0]
    assert resumed[1] == 0
    assert s_small.counters["preemptions"] >= 1
    assert not s_small.requests and not s_big.requests, "finished requests leave the scheduler's table"


def test_resumed_requests_are_preempted_last():
    m, s = make(num_blocks=64, bs=4, max_seqs=4)
    for i in range(3):
        s.add(f"r{i}", [1, 2, 3], SamplingParams(max_tokens=50), seed=i)
    run_step(m, s)
    s.requests["r2"].resumed = True
    victims = sorted(s.running, key=lambda r: (r.resumed, -r.arrival))
    assert [r.rid for r in victims] == ["r1", "r0", "r2"]


def test_lone_request_that_outgrows_the_cache_ends():
    m, s = make(num_blocks=3, bs=4)             # 12 tokens
    s.add("a", [1] * 5, SamplingParams(max_tokens=100), seed=0)
    outs = drive(m, s)
    assert outs["a"][1] == "cache" and len(outs["a"][0]) == 8      # 5 + 7 fill the 12 slots; the 8th token has no slot
    assert all(p.num_free == p.num_blocks for p in m.pools)


def test_abort_is_idempotent_and_isolated():
    def run(abort):
        m, s = make()
        for i in range(3):
            s.add(f"r{i}", [i + 1] * 5, SamplingParams(max_tokens=12), seed=i)
        run_step(m, s)
        run_step(m, s)
        if abort:
            r1 = s.requests["r1"]
            assert s.abort("r1") and not s.abort("r1") and not s.abort("nobody")
            assert r1.finish_reason == "abort" and "r1" not in s.requests
        outs = drive(m, s)
        m.check()
        assert all(p.num_free == p.num_blocks for p in m.pools)
        return outs
    with_abort, without = run(True), run(False)
    assert "r1" not in with_abort
    assert with_abort["r0"] == without["r0"] and with_abort["r2"] == without["r2"]
    # aborting a waiting request
    m, s = make(max_seqs=1)
    s.add("a", [1], SamplingParams(max_tokens=3), seed=0)
    b = s.add("b", [1], SamplingParams(max_tokens=3), seed=0)
    assert s.abort("b") and b.state == FINISHED and "b" not in s.requests
    assert set(drive(m, s)) == {"a"}


def test_max_num_seqs_caps_running():
    m, s = make(max_seqs=2)
    for i in range(5):
        s.add(f"r{i}", [1, 2], SamplingParams(max_tokens=3), seed=i)
    while s.has_work():
        run_step(m, s)
        assert len(s.running) <= 2
    assert s.counters["finished"] == 5


def test_admission_keeps_headroom_for_running_requests():
    m, s = make(num_blocks=6, bs=4, budget=64)
    s.add("a", [1] * 8, SamplingParams(max_tokens=20), seed=0)
    run_step(m, s)                              # a holds 2 blocks (+1 at its next token)
    s.add("b", [1] * 16, SamplingParams(max_tokens=2), seed=0)
    plan, _ = run_step(m, s)
    # 4 blocks free, a takes 1, one stays in reserve for a: b gets 2 blocks = 8 tokens now
    assert [(p.request.rid, p.start, p.length) for p in plan.portions] == [("a", 8, 1), ("b", 0, 8)]


def test_replay_twice_is_identical():
    """A fixed arrival list decides the same twice (crates/scheduler/src/replay.rs:171-177)."""
    def run(seed):
        import random
        rng = random.Random(seed)
        m, s = make(num_blocks=24, bs=4, budget=24, max_seqs=4, windows=(0, 6))
        arrivals = [(rng.randrange(0, 30), [rng.randrange(1, 99) for _ in range(rng.randrange(1, 30))],
                     rng.randrange(1, 20)) for _ in range(12)]
        log, outs, step, i = [], {}, 0, 0
        arrivals.sort(key=lambda a: a[0])
        while i < len(arrivals) or s.has_work():
            while i < len(arrivals) and arrivals[i][0] <= step:
                s.add(f"r{i}", arrivals[i][1], SamplingParams(max_tokens=arrivals[i][2]), seed=i)
                i += 1
            if s.has_work():
                plan, done = run_step(m, s, log)
                for r in done + plan.finished:
                    outs[r.rid] = (list(r.output), r.finish_reason)
            step += 1
            assert step < 5000
        assert all(p.num_free == p.num_blocks for p in m.pools)
        return log, outs
    for seed in range(5):
        assert run(seed) == run(seed)


def test_stop_sequences_fire_on_the_generated_suffix():
    """The reference's matcher cases (crates/scheduler/src/stop.rs:97-158) through the scheduler:
    a pattern spanning steps, a mismatch that resets, 'aaa' on a stream of a's, overlapping
    patterns, an empty pattern. The last token of the match is consumed, the ones before it
    were emitted; the prompt is no part of the stream."""
    def run(stream, patterns, prompt=(1,)):
        m, s = make()
        s.add("a", list(prompt), SamplingParams(max_tokens=50, ignore_eos=True, stop_sequences=patterns), seed=0)
        it = iter(stream)
        return drive(m, s, token_fn=lambda rid, pos: next(it))["a"]
    assert run([1, 7, 9], ((7,),)) == ([1], "stop")
    assert run([3, 1, 9, 3, 1, 4, 8], ((3, 1, 4),)) == ([3, 1, 9, 3, 1], "stop")
    assert run([1, 2, 1, 3, 1, 2, 1, 2, 5], ((1, 2, 1, 2),)) == ([1, 2, 1, 3, 1, 2, 1], "stop")
    assert run([5, 5, 5, 5], ((5, 5, 5),)) == ([5, 5], "stop")
    assert run([1, 2, 3, 4], ((1, 2, 3), (2, 3))) == ([1, 2], "stop")
    assert run([6, 4, 2], ((), (4,))) == ([6], "stop")
    # the prompt's tokens do not count: 3 1 in the prompt, 4 generated first
    assert run([4, 3, 1, 4, 0], ((3, 1, 4),), prompt=(3, 1)) == ([4, 3, 1], "stop")


# ---------------------------------------------------------------- admission by the estimated peak
def test_peak_formula_and_estimates():
    """max over k of b[k] (k + 1) + a[0..k], sorted by b descending (crates/scheduler/src/admission.rs:138-148):
    the cases are worked by hand."""
    assert Scheduler.peak_tokens([]) == 0
    assert Scheduler.peak_tokens([(10, 5)]) == 15
    # b descending: (10, 30), (100, 20), (50, 1): 30 + 10 = 40; 20 * 2 + 110 = 150; 1 * 3 + 160 = 163
    assert Scheduler.peak_tokens([(100, 20), (50, 1), (10, 30)]) == 163
    # one long request beside short ones: the peak is while all are there, not the sum of all ends
    assert Scheduler.peak_tokens([(10, 100), (10, 2), (10, 2)]) == max(100 + 10, 2 * 2 + 20, 2 * 3 + 30)
    m, s = make(num_blocks=1024, bs=4, max_model_len=4096, admission="peak")
    r = s.add("a", [1] * 20, SamplingParams(max_tokens=300), seed=0)
    assert s.ema_out == 2048.0
    assert s.estimate(r) == (21, 300 + 16)                 # not busy: min(cap, max(1.1 * 0, mean)) + 16
    s.observe_output(100)                                   # falls with weight 0.4 on what was seen
    assert abs(s.ema_out - (0.6 * 2048 + 0.4 * 100)) < 1e-9
    for _ in range(40):
        s.observe_output(10)
    assert s.ema_out == 64.0                                # never below 64
    assert s.estimate(r) == (21, 64 + 16)
    assert s.estimate(r, busy=True) == (21, 300 + 16)       # busy: all it may
    while len(r.output) < 100:
        run_step(m, s)
    import math
    assert s.estimate(r) == (121, math.ceil(1.1 * 100) - 100 + 16)      # 1.1 x what it has generated, less what it has
    s.observe_output(1000)                                  # rises with weight 0.1
    assert abs(s.ema_out - (0.9 * 64 + 0.1 * 1000)) < 1e-9


def test_peak_admission_holds_back_instead_of_preempting():
    """64 tokens of cache for three requests of about 39: admitted by blocks they preempt each
    other; admitted by the estimate they run one after the other, nothing is recomputed, and the
    outputs are the same. Arrival order is kept: nobody overtakes the request that is held back."""
    def run(admission):
        m, s = make(num_blocks=16, bs=4, budget=64, max_seqs=4, admission=admission)
        for i, n in enumerate([9, 7, 8]):
            s.add(f"r{i}", list(range(1, n + 1)), SamplingParams(max_tokens=30), seed=i)
        log = []
        outs = drive(m, s, log)
        assert all(p.num_free == p.num_blocks for p in m.pools)
        return outs, log, s
    by_blocks, _, s_blocks = run("blocks")
    by_peak, log, s_peak = run("peak")
    assert by_peak == by_blocks
    assert s_blocks.counters["preemptions"] > 0
    assert s_peak.counters["preemptions"] == 0 and s_peak.counters["held_back"] > 0
    assert s_peak.counters["tokens"] == sum(n + 29 for n in (9, 7, 8)), "every token computed once"
    first_seen = []
    for portions, _ in log:
        for rid, _, _ in portions:
            if rid not in first_seen:
                first_seen.append(rid)
    assert first_seen == ["r0", "r1", "r2"]


def test_peak_admission_lets_in_what_fits_and_a_lone_request_always():
    m, s = make(num_blocks=64, bs=4, budget=256, max_seqs=8, admission="peak")      # 256 tokens
    for _ in range(8):
        s.observe_output(8)                                 # the mean of finished outputs comes down to its floor of 64
    for i in range(4):
        s.add(f"r{i}", [1] * 20, SamplingParams(max_tokens=40), seed=i)
    plan, _ = run_step(m, s)
    # (a, b) = (21, 56) each; the pool less a partly empty block a request: k requests need 56 k + 21 k + 3 k <= 256
    assert [p.request.rid for p in plan.portions] == ["r0", "r1", "r2"]
    assert s.counters["held_back"] == 1
    # a request larger than the estimate allows still runs when it is alone
    m2, s2 = make(num_blocks=16, bs=4, budget=64, admission="peak")
    s2.add("big", [1] * 30, SamplingParams(max_tokens=500), seed=0)
    plan, _ = run_step(m2, s2)
    assert [(p.request.rid, p.length) for p in plan.portions] == [("big", 30)]


def test_peak_admission_is_deterministic_and_complete():
    import random
    def run():
        rng = random.Random(5)
        m, s = make(num_blocks=40, bs=4, budget=48, max_seqs=6, admission="peak")
        for i in range(30):
            s.add(f"r{i}", [1 + i] * rng.randint(1, 60), SamplingParams(max_tokens=rng.randint(1, 40)), seed=i)
        log = []
        outs = drive(m, s, log)
        return outs, log, dict(s.counters)
    a, b = run(), run()
    assert a == b
    assert len(a[0]) == 30 and all(reason == "length" for _, reason in a[0].values())


def test_prompts_that_fill_the_pool_between_them_do_not_stall():
    """Admission by free blocks with portions smaller than the budget lets two long prompts in side
    by side; when the pool is full and neither has reached its end, nobody decodes, so nobody makes
    room: the newest goes back to the queue and the older one finishes first."""
    m, s = make(num_blocks=32, bs=4, budget=32, max_chunk=16, admission="blocks")
    s.add("a", list(range(1, 101)), SamplingParams(max_tokens=4), seed=0)
    s.add("b", list(range(1, 101)), SamplingParams(max_tokens=4), seed=1)
    log = []
    outs = drive(m, s, log, limit=200)
    assert set(outs) == {"a", "b"} and all(len(o) == 4 and why == "length" for o, why in outs.values())
    assert s.counters["preemptions"] >= 1
    assert any("b" in pre for _, pre in log), "the newer request is the one that goes back"
    assert all(p.num_free == p.num_blocks for p in m.pools)
    # the same requests with room for both give the same tokens
    m2, s2 = make(num_blocks=64, bs=4, budget=32, max_chunk=16, admission="blocks")
    s2.add("a", list(range(1, 101)), SamplingParams(max_tokens=4), seed=0)
    s2.add("b", list(range(1, 101)), SamplingParams(max_tokens=4), seed=1)
    assert drive(m2, s2) == outs


def test_finished_requests_are_forgotten():
    m, s = make()
    held = [s.add(f"r{i}", [1, 2, 3], SamplingParams(max_tokens=3), seed=i) for i in range(6)]
    drive(m, s)
    assert len(s.requests) == 0
    assert all(r.state == FINISHED and len(r.output) == 3 for r in held)     # the caller's objects live on
    s.add("r0", [1, 2, 3], SamplingParams(max_tokens=1), seed=0)             # an id may be used again
    assert set(drive(m, s)) == {"r0"}


def drive_one_step_late(m, s, token_fn=fake_token, aborts=None, limit=10000):
    """The loop of the engine that launches a step before it has read the tokens of the step before:
    schedule, launch (here: take the blocks), advance blind, and only then resolve the step before."""
    outs, pending, n = {}, None, 0
    aborts = dict(aborts or {})
    while s.has_work() or pending is not None:
        plan = s.schedule()
        for r in plan.finished:
            outs[r.rid] = (list(r.output), r.finish_reason)
        live = [p for p in plan.portions if p.request.state == RUNNING]
        for p in live:
            assert p.start == p.request.num_computed
            m.grow(p.request.rid, p.start + p.length)
        for p in live:
            m.commit(p.request.rid, p.start + p.length)
        tokens = [token_fn(p.request.rid, p.request.num_tokens) for p in live if p.samples]
        s.advance_blind(plan)
        if pending is not None:
            for r in s.resolve(*pending):
                outs[r.rid] = (list(r.output), r.finish_reason)
        pending = (plan, tokens) if live else None
        for rid in aborts.pop(n, []):
            s.abort(rid)
        m.check()
        n += 1
        assert n < limit, "the scheduler does not terminate"
    return outs


@pytest.mark.parametrize("seed", range(6))
def test_tokens_read_one_step_late_change_nothing(seed):
    """Requests whose tokens are read a step late (the next step is planned and launched first) end with the
    tokens and reasons of the loop that reads at once: a stop token cuts off the place that the later step
    had already added, the cap and the context end a request at launch time, a stop at the very last token
    still wins over the cap; under preemptions (a pool too small for all) and with stop sequences."""
    import random
    rng = random.Random(seed)
    reqs = []
    for i in range(14):
        stops = ([rng.randrange(20)] if rng.random() < 0.5 else [])
        seqs = ([[rng.randrange(20), rng.randrange(20)]] if rng.random() < 0.4 else [])
        reqs.append((f"r{i}", [rng.randrange(1000) for _ in range(rng.randrange(1, 40))],
                     SamplingParams(max_tokens=rng.randrange(1, 30), stop_token_ids=stops, stop_sequences=seqs)))

    def tok(rid, position):
        return fake_token(rid, position, vocab=20)          # few values: stops and stop sequences do fire

    results = []
    for driver in (drive, drive_one_step_late):
        m, s = make(num_blocks=30, bs=4, max_seqs=5, budget=24, max_chunk=12, eos=(7,), max_model_len=60)
        for rid, prompt, params in reqs:
            s.add(rid, prompt, params, seed=0)
        outs = driver(m, s, token_fn=tok)
        assert all(p.num_free == p.num_blocks for p in m.pools)
        assert not s.running and not s.waiting
        results.append((outs, s.counters["preemptions"]))
    assert results[0][0] == results[1][0]
    reasons = {r for _, r in results[0][0].values()}
    assert {"stop", "length"} <= reasons, reasons


def test_abort_and_stop_while_a_step_is_in_flight():
    m, s = make(num_blocks=40, bs=4, eos=(5,))
    for i in range(3):
        s.add(f"r{i}", [1, 2, 3], SamplingParams(max_tokens=20), seed=0)
    # r1's second token is the end-of-sequence id; r2 is aborted while a step with its row is in flight
    def tok(rid, position):
        return 5 if (rid, position) == ("r1", 4) else 100 + position
    outs = drive_one_step_late(m, s, token_fn=tok, aborts={2: ["r2"]})
    assert outs["r1"] == ([103], "stop")
    assert outs["r0"][1] == "length" and outs["r0"][0] == [100 + p for p in range(3, 23)]
    assert "r2" not in outs                     # an aborted request is not reported as done
    assert all(p.num_free == p.num_blocks for p in m.pools)
    assert s.counters["finished"] == 2
