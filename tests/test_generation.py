"""Generation through the Python entry point and the command line: greedy equals the
plain implementation, preemption does not change outputs, seeded temperature
sampling does not depend on the batch. The CPU runs use the kernel stand-in
(bookkeeping only); the ``gpu`` runs use the real kernels."""
import json
import os
import subprocess
import sys

import pytest
import torch

import plain_qwen3 as plain
from helpers import TINY, make_folder, random_tokens, read_folder
from kernel_double import KernelDouble
from reinfer_amd import LLMEngine, SamplingParams, kernels

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def engine_for(folder, device, dtype="float32", **kw):
    return LLMEngine(folder, dtype=dtype, device=device, **kw)


def check_greedy(folder, device):
    raw, w = read_folder(folder)
    prompts = [random_tokens(n, raw["vocab_size"], 40 + n) for n in (5, 17, 33)]
    want = [plain.greedy_generate(raw, w, p, 16) for p in prompts]
    eng = engine_for(folder, device, num_blocks=32)
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=16))
    assert [o.token_ids for o in outs] == want
    assert all(o.finish_reason == "length" for o in outs)
    # so few blocks that requests are preempted and recomputed: the same tokens
    small = engine_for(folder, device, num_blocks=6, max_num_batched_tokens=24, admission="blocks")
    outs2 = small.generate(prompts, SamplingParams(temperature=0.0, max_tokens=16))
    assert [o.token_ids for o in outs2] == want
    assert small.cache_stats()["preemptions"] > 0
    assert small.cache_stats()["blocks_free"] == small.cache_stats()["blocks_total"]
    # the same pool with admission by the estimated peak: requests wait instead, nothing is recomputed
    held = engine_for(folder, device, num_blocks=6, max_num_batched_tokens=24)
    outs3 = held.generate(prompts, SamplingParams(temperature=0.0, max_tokens=16))
    assert [o.token_ids for o in outs3] == want
    assert held.cache_stats()["preemptions"] == 0 and held.cache_stats()["held_back"] > 0
    return eng


def check_temperature(folder, device):
    raw, w = read_folder(folder)
    V = raw["vocab_size"]
    prompts = [random_tokens(n, V, 70 + n) for n in (1, 7, 64, 130)]
    sp = [SamplingParams(temperature=0.8, seed=1000 + i, max_tokens=12) for i in range(len(prompts))]
    eng = engine_for(folder, device, num_blocks=64, max_num_batched_tokens=16)    # portions of 16 beside decodes
    together = [o.token_ids for o in eng.generate(prompts, sp)]
    again = [o.token_ids for o in eng.generate(prompts, sp)]
    assert together == again, "same seed, same tokens"
    alone = [eng.generate([p], s)[0].token_ids for p, s in zip(prompts, sp)]
    assert alone == together, "a request's tokens do not depend on the batch"
    other = eng.generate(prompts[:1], SamplingParams(temperature=0.8, seed=5, max_tokens=12))[0].token_ids
    assert other != together[0]
    assert all(0 <= t < V for o in together for t in o)


def test_greedy_generation_cpu_bookkeeping(tmp_path):
    with kernels.use(KernelDouble()):
        check_greedy(make_folder(tmp_path, "A", "float32"), "cpu")


def test_temperature_generation_cpu_bookkeeping(tmp_path):
    with kernels.use(KernelDouble()):
        check_temperature(make_folder(tmp_path, "B", "float32"), "cpu")


def test_eos_from_config_stops_generation(tmp_path):
    with kernels.use(KernelDouble()):
        folder = make_folder(tmp_path, "A", "float32")
        raw, w = read_folder(folder)
        prompt = random_tokens(6, raw["vocab_size"], 5)
        free_run = plain.greedy_generate(raw, w, prompt, 6)
        raw2 = dict(raw, eos_token_id=free_run[3])
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(raw2, f)
        out = engine_for(folder, "cpu", num_blocks=16).generate([prompt], SamplingParams(max_tokens=6))[0]
        cut = free_run.index(free_run[3])
        assert out.token_ids == free_run[:cut] and out.finish_reason == "stop"


@pytest.mark.gpu
@pytest.mark.parametrize("which", ["A", "C"])
def test_greedy_generation_gpu(tmp_path, which):
    eng = check_greedy(make_folder(tmp_path, which, "float32"), "cuda:0")
    assert kernels.current().name == "hip-gfx950"


@pytest.mark.gpu
def test_temperature_generation_gpu(tmp_path):
    check_temperature(make_folder(tmp_path, "B", "float32"), "cuda:0")


@pytest.mark.gpu
def test_bfloat16_greedy_mostly_agrees_with_plain(tmp_path):
    """bfloat16 may flip a near tie; where the plain top-2 gap is clear the tokens agree. Clear: more than
    twice the bound on a bfloat16 logit's error (helpers.TOL of the largest logit), so that no rounding
    within the bound can change the order. Enough positions must have such a gap for the test to say
    anything."""
    from helpers import TOL
    folder = make_folder(tmp_path, "B", "bfloat16")
    raw, w = read_folder(folder)
    eng = engine_for(folder, "cuda:0", dtype="bfloat16", num_blocks=64)
    compared = 0
    for seed in (9, 10, 11, 12):
        prompt = random_tokens(20, raw["vocab_size"], seed)
        out = eng.generate([prompt], SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True))[0].token_ids
        assert len(out) == 12
        toks = list(prompt)
        for t in out:
            logits = plain.forward(raw, w, toks)[-1]
            top2 = torch.topk(logits, 2).values
            if (top2[0] - top2[1]) > 2.0 * TOL["bfloat16"] * logits.abs().max():
                assert t == int(torch.argmax(logits))
                compared += 1
            toks.append(t)
    assert compared >= 8, f"only {compared} of 48 positions had a clear gap"


@pytest.mark.gpu
def test_command_line_run(tmp_path):
    folder = make_folder(tmp_path, "A", "float32")
    raw, w = read_folder(folder)
    prompt = [3, 141, 59, 26, 53]
    want = plain.greedy_generate(raw, w, prompt, 8)
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "reinfer"), "run", folder, "-n", "8", "-t", "0",
                        "--dtype", "float32", "--num-blocks", "16", "--perf", "--"] + [str(t) for t in prompt],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert [int(t) for t in r.stdout.split()] == want
    assert "PERF " in r.stderr and "tok_s=" in r.stderr and "first_token_ms=" in r.stderr


def test_command_line_backend_option():
    """`run m --backend bogus` is a usage error and the default is auto
    (bin/reinfer/src/main.rs:2135-2140); here the only backends are auto and hip."""
    from reinfer_amd import cli
    with pytest.raises(SystemExit) as e:
        cli.main(["run", "m", "--backend", "bogus"])
    assert e.value.code == 2
    with pytest.raises(SystemExit):
        cli.main(["run", "m", "--backend", "cuda"])
    assert cli._backend("auto") == "auto" and cli._backend("hip") == "hip"


def test_command_line_bench_passes_options_on():
    """`reinfer bench --gpus 2` hands everything behind the verb to bench.py, options first or not:
    bench.py says that it runs on one GPU and the exit status is its 2."""
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "reinfer"), "bench", "--gpus", "2"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 2 and "one GPU" in r.stdout


@pytest.mark.gpu
def test_many_requests_with_mixed_sampling_do_not_depend_on_the_batch(tmp_path):
    """Forty requests of many lengths and caps, greedy beside temperature, top-k / top-p, min-p with a
    repeat penalty and stop ids: run together (portions of 96 tokens beside up to 32 decoding requests),
    each alone, and together in a pool so small that requests are preempted and recomputed. In 32-bit
    every kernel sums in a fixed order, so the tokens and the finish reasons are the same."""
    import random
    folder = make_folder(tmp_path, "C", "float32")
    raw, _ = read_folder(folder)
    V = raw["vocab_size"]
    rng = random.Random(1)
    prompts, params = [], []
    for i in range(40):
        prompts.append(random_tokens(rng.choice([1, 2, 5, 17, 33, 64, 65, 100, 130]), V, 1000 + i))
        cap = rng.choice([1, 2, 7, 30, 60])
        params.append([SamplingParams(temperature=0.0, max_tokens=cap),
                       SamplingParams(temperature=0.8, seed=50 + i, max_tokens=cap),
                       SamplingParams(temperature=0.9, seed=50 + i, top_k=20, top_p=0.9, max_tokens=cap),
                       SamplingParams(temperature=0.7, seed=50 + i, min_p=0.05, repeat_penalty=1.2, max_tokens=cap,
                                      stop_token_ids=[3, 4, 5])][i % 4])
    limits = dict(max_num_batched_tokens=96, max_model_len=250)
    eng = engine_for(folder, "cuda:0", num_blocks=200, max_num_seqs=32, **limits)
    together = eng.generate(prompts, params)
    assert eng.cache_stats()["blocks_free"] == eng.cache_stats()["blocks_total"]
    one = engine_for(folder, "cuda:0", num_blocks=32, max_num_seqs=2, **limits)
    for i, (p, sp) in enumerate(zip(prompts, params)):
        alone = one.generate([p], sp)[0]
        assert (alone.token_ids, alone.finish_reason) == (together[i].token_ids, together[i].finish_reason), i
    small = engine_for(folder, "cuda:0", num_blocks=40, max_num_seqs=32, admission="blocks", **limits)
    again = small.generate(prompts, params)
    assert small.cache_stats()["preemptions"] > 0
    assert [o.token_ids for o in again] == [o.token_ids for o in together]


@pytest.mark.gpu
def test_aborts_and_arrivals_between_captured_decode_steps(tmp_path):
    """Requests are aborted and others arrive while the rest decode from captured steps: the rows of
    a captured step change hands (another request, another block table), a request id comes back from
    its start, every block returns, and in 32-bit each finished request has the tokens it has alone."""
    folder = make_folder(tmp_path, "B", "float32")
    raw, _ = read_folder(folder)
    V = raw["vocab_size"]
    P = {k: random_tokens(n, V, 10 + i) for i, (k, n) in enumerate((("a", 20), ("b", 35), ("c", 9), ("d", 50), ("e", 28), ("f", 3)))}
    sp = SamplingParams(temperature=0.0, max_tokens=40)
    one = engine_for(folder, "cuda:0", num_blocks=64, max_num_seqs=2)
    alone = {k: one.generate([p], sp)[0].token_ids for k, p in P.items()}
    eng = engine_for(folder, "cuda:0", num_blocks=64, max_num_seqs=8)
    for k in "abcd":
        eng.add_request(P[k], sp, rid=k)
    outs, step = {}, 0
    while eng.has_unfinished():
        for o in eng.step():
            outs[o.rid] = o
        step += 1
        if step == 8:
            assert eng.abort("b") and not eng.abort("b")
            eng.add_request(P["e"], sp, rid="e")
        if step == 15:
            assert eng.abort("a")
            eng.add_request(P["f"], sp, rid="f")
            eng.add_request(P["b"], sp, rid="b")
    assert sorted(outs) == ["b", "c", "d", "e", "f"]
    assert {k: outs[k].token_ids for k in outs} == {k: alone[k] for k in outs}
    assert eng.runner.graphs is not None and eng.runner.graphs.replays > 30
    assert eng.cache_stats()["blocks_free"] == eng.cache_stats()["blocks_total"]


@pytest.mark.gpu
def test_a_token_that_ends_a_request_is_read_one_step_late(tmp_path):
    """Decode steps are launched before the tokens of the step before have been read: a request that its
    end-of-sequence id ended has one more row in flight by then. Several requests decode together, the id ends
    them at different steps: each has the tokens of the plain loop up to (not including) the id, the others go
    on undisturbed, every block comes back."""
    folder = make_folder(tmp_path, "A", "float32")
    raw, w = read_folder(folder)
    prompts = [random_tokens(n, raw["vocab_size"], 60 + n) for n in (6, 11, 19, 4)]
    free = [plain.greedy_generate(raw, w, p, 14) for p in prompts]
    eos = free[0][3]
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(dict(raw, eos_token_id=eos), f)
    eng = engine_for(folder, "cuda:0", num_blocks=32)
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=14))
    for run, o in zip(free, outs):
        want = run[:run.index(eos)] if eos in run else run
        assert o.token_ids == want
        assert o.finish_reason == ("stop" if eos in run else "length")
    assert outs[0].finish_reason == "stop" and any(o.finish_reason == "length" for o in outs)
    assert eng.runner.graphs is not None and eng.runner.graphs.replays >= 10
    assert eng.cache_stats()["blocks_free"] == eng.cache_stats()["blocks_total"]
    assert not eng.has_unfinished()


@pytest.mark.gpu
@pytest.mark.parametrize("seed", [2, 37, 56])
def test_steps_launched_one_ahead_give_what_steps_resolved_at_once_give(tmp_path, seed):
    """Random requests (lengths, temperatures, seeds, stop ids, caps, top-k) under random limits (blocks, running
    requests, step budget, admission; seeds 37 and 56 preempt): once as the engine runs them, decode steps
    launched before the tokens of the step before are read, once with every step resolved before the next
    is planned. The same tokens and the same reasons for ending, and every block back."""
    import random
    rng = random.Random(seed)
    which = rng.choice("ABC")
    dtype = rng.choice(["bfloat16", "float32"])
    folder = make_folder(tmp_path, which, dtype)
    raw, _ = read_folder(folder)
    V = raw["vocab_size"]
    n = rng.randrange(4, 40)
    prompts = [random_tokens(rng.randrange(2, 90), V, 1000 * seed + i) for i in range(n)]
    params = []
    for i in range(n):
        stops = tuple(rng.randrange(V) for _ in range(rng.choice([0, 0, 3, 40])))
        params.append(SamplingParams(temperature=rng.choice([0.0, 0.0, 0.7, 1.3]), seed=rng.randrange(1 << 30),
                                     max_tokens=rng.randrange(1, 60), stop_token_ids=stops,
                                     top_k=rng.choice([None, None, 5]), ignore_eos=rng.random() < 0.5))
    kw = dict(num_blocks=rng.choice([24, 40, 200]), max_num_seqs=rng.choice([4, 16, 64]),
              max_num_batched_tokens=rng.choice([32, 64, 256]), admission=rng.choice(["peak", "blocks"]))
    outs = {}
    for mode in ("ahead", "at once"):
        eng = engine_for(folder, "cuda:0", dtype=dtype, **kw)
        if mode == "at once":
            eng.runner.can_chain = lambda rows: False
        res = eng.generate(prompts, params)
        outs[mode] = [(o.token_ids, o.finish_reason) for o in res]
        stats = eng.cache_stats()
        assert stats["blocks_free"] == stats["blocks_total"]
        if mode == "ahead":
            assert eng.runner.graphs is not None and eng.runner.graphs.replays > 0
    assert outs["ahead"] == outs["at once"]
    assert {r for _, r in outs["ahead"]} >= {"length"}
