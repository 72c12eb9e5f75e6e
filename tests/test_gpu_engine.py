"""The engine on the GPU against the plain implementation, in 32-bit and bfloat16:
whole requests, most in one step and the last 32 tokens one by one, portions of
changing size, mixed batches with page reuse, long decoding, the first tokens.
The logits at a position must not depend on how the tokens were cut into steps,
on what else is in the batch or on which blocks are used, beyond rounding."""
import pytest
import torch

import plain_qwen3 as plain
from helpers import TINY, TOL, make_folder, mixed_plan, random_tokens, read_folder, rel_err, run_plan
from reinfer_amd import kernels
from reinfer_amd.engine import ModelRunner, StepEntry

pytestmark = pytest.mark.gpu

CASES = [(w, d) for w in ("A", "B", "C") for d in ("float32", "bfloat16")]


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("models")
    return {(w, d): make_folder(base, w, d) for w, d in CASES}


@pytest.fixture(scope="module")
def plain_cache():
    return {}


def reference(folders, plain_cache, which, dtype, toks):
    key = (which, dtype, tuple(toks))
    if key not in plain_cache:
        raw, weights = read_folder(folders[(which, dtype)])
        plain_cache[key] = plain.forward(raw, weights, toks).float()
    return plain_cache[key]


def runner_for(folders, which, dtype, **limits):
    assert kernels.current().name == "hip-gfx950"
    return ModelRunner.from_folder(folders[(which, dtype)], dtype=dtype, device="cuda:0", **limits)


def vocab(which):
    return TINY[which][0]["vocab_size"]


@pytest.mark.parametrize("which,dtype", CASES)
def test_whole(folders, plain_cache, which, dtype):
    runner = runner_for(folders, which, dtype, max_tokens=256)
    for n, seed in ((5, 1), (17, 2), (33, 3), (130, 4), (1, 5)):
        toks = random_tokens(n, vocab(which), seed)
        got = run_plan(runner, {"r": toks}, [[("r", n)]])["r"]
        assert rel_err(got, reference(folders, plain_cache, which, dtype, toks)) < TOL[dtype], (n,)
    assert all(p.num_free == p.num_blocks for p in runner.manager.pools)


@pytest.mark.parametrize("which,dtype", CASES)
def test_last_32_one_by_one(folders, plain_cache, which, dtype):
    runner = runner_for(folders, which, dtype, max_tokens=256)
    n = 150
    toks = random_tokens(n, vocab(which), 21)
    plan = [[("r", n - 32)]] + [[("r", 1)]] * 32
    got = run_plan(runner, {"r": toks}, plan)["r"]
    assert rel_err(got, reference(folders, plain_cache, which, dtype, toks)) < TOL[dtype]


@pytest.mark.parametrize("which,dtype", CASES)
def test_portions_of_changing_size(folders, plain_cache, which, dtype):
    runner = runner_for(folders, which, dtype, max_tokens=256)
    n = 131
    toks = random_tokens(n, vocab(which), 22)
    cuts = [7, 2, 16, 3, 2, 17, 2, 31, 2, 15, 1, 16, 2, 2, 13]
    assert sum(cuts) == n
    got = run_plan(runner, {"r": toks}, [[("r", c)] for c in cuts])["r"]
    assert rel_err(got, reference(folders, plain_cache, which, dtype, toks)) < TOL[dtype]


@pytest.mark.parametrize("which,dtype", CASES)
def test_mixed_with_page_reuse(folders, plain_cache, which, dtype):
    runner = runner_for(folders, which, dtype, max_tokens=128)
    lens, plan = mixed_plan()
    seqs = {r: random_tokens(n, vocab(which), 300 + i) for i, (r, n) in enumerate(lens.items())}
    # poison everything a request does not own: a read outside its blocks shows as NaN
    for c in runner.caches:
        if c is not None and c.k is not None:
            c.k.fill_(float("nan"))
            c.v.fill_(float("nan"))
    runner.poison_freed_blocks()           # and again whenever a block goes back: a freed slot reads NaN, not stale values
    got = run_plan(runner, seqs, plan)
    for r, toks in seqs.items():
        assert rel_err(got[r], reference(folders, plain_cache, which, dtype, toks)) < TOL[dtype], r
    pool = runner.manager.pools[0]
    assert pool.allocs > pool.num_blocks, "the plan must reuse blocks"


@pytest.mark.parametrize("which,dtype", [("A", "float32"), ("B", "bfloat16"), ("C", "bfloat16")])
def test_long_decoding(folders, plain_cache, which, dtype):
    runner = runner_for(folders, which, dtype, max_tokens=256)
    n = 200
    toks = random_tokens(n, vocab(which), 23)
    got = run_plan(runner, {"r": toks}, [[("r", 3)]] + [[("r", 1)]] * (n - 3))["r"]
    assert rel_err(got, reference(folders, plain_cache, which, dtype, toks)) < TOL[dtype]


@pytest.mark.parametrize("which,dtype", CASES)
def test_first_tokens(folders, plain_cache, which, dtype):
    """Positions 0, 1, 2 on their own: one key, two keys; page edges at 15/16/17."""
    runner = runner_for(folders, which, dtype, max_tokens=64)
    toks = random_tokens(18, vocab(which), 24)
    ref = reference(folders, plain_cache, which, dtype, toks)
    got = run_plan(runner, {"r": toks}, [[("r", 1)]] * 18)["r"]
    assert rel_err(got[:3], ref[:3]) < TOL[dtype]
    assert rel_err(got, ref) < TOL[dtype]


def test_far_key_stands_out(folders):
    """One early key that a late query must find among hundreds: a fault in the
    block table walk or in the running maximum would lose it. The query and key
    weights of the first layer are scaled so that scores are sharp."""
    which, dtype = "B", "float32"
    raw, weights = read_folder(folders[(which, dtype)])
    weights = {k: v.clone() for k, v in weights.items()}
    for name in ("q_norm", "k_norm"):
        weights[f"model.layers.0.self_attn.{name}.weight"] *= 3.0
    from reinfer_amd.config import config_from_dict
    runner = ModelRunner.from_config(config_from_dict(raw), dtype=dtype, weights=weights, max_tokens=512)
    toks = random_tokens(400, raw["vocab_size"], 25)
    ref = plain.forward(raw, weights, toks).float()
    plan = [[("r", 2)], [("r", 333)], [("r", 2)]] + [[("r", 1)]] * 63
    got = run_plan(runner, {"r": toks}, plan)["r"]
    assert rel_err(got, ref) < TOL[dtype]


def test_batch_order_does_not_matter(folders):
    runner = runner_for(folders, "A", "float32", max_tokens=256)
    V = vocab("A")
    seqs = {"x": random_tokens(30, V, 31), "y": random_tokens(9, V, 32), "z": random_tokens(17, V, 33)}
    a = run_plan(runner, seqs, [[("x", 30), ("y", 9), ("z", 17)]])
    b = run_plan(runner, seqs, [[("z", 17), ("x", 30), ("y", 9)]])
    alone = {r: run_plan(runner, {r: t}, [[(r, len(t))]])[r] for r, t in seqs.items()}
    for r in seqs:
        assert rel_err(a[r], alone[r]) < 1e-5
        assert rel_err(b[r], alone[r]) < 1e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_whose_logits_nobody_reads(folders, plain_cache, dtype):
    """Single-token steps with nothing wanted, between steps that are read: nobody waits for such a
    step's results, so the next step is packed while it may not have started; each must still run with
    its own indices (the steps replay a captured graph from a staging buffer that is written again)."""
    toks = random_tokens(90, vocab("B"), 77)
    want = reference(folders, plain_cache, "B", dtype, toks)
    runner = runner_for(folders, "B", dtype, max_tokens=512, max_seqs=4)
    for rep in range(2):                       # the second request replays the graph the first captured
        runner.add_request("x")
        runner.step([StepEntry("x", toks[:40], [])])
        got = {}
        for p in range(40, 90):
            out = runner.step([StepEntry("x", [toks[p]], [0] if p % 7 == 0 or p == 89 else [])])
            if out.shape[0]:
                got[p] = out[0].float().cpu()
        runner.free_request("x")
        assert len(got) == 8
        for p, row in got.items():
            assert rel_err(row[None], want[p][None]) < TOL[dtype], (rep, p)



@pytest.mark.parametrize("which,n_req", [("A", 5), ("B", 70)])
def test_decode_graphs_replay_like_eager_steps(folders, which, n_req):
    """Decode steps replay captured HIP graphs (one per batch-size and context bucket, library
    products included above 64 rows). Every replay is checked against a runner that launches the
    same step kernel by kernel: the same bucket several times, with prompt steps (eager work and
    synchronisations) between the replays, requests leaving, and a second context bucket."""
    dtype = "bfloat16"
    V = vocab(which)
    with_graphs = runner_for(folders, which, dtype, max_tokens=n_req * 320, max_seqs=128)
    eager = runner_for(folders, which, dtype, max_tokens=n_req * 320, max_seqs=128, use_graphs=False)
    assert with_graphs.graphs is not None and eager.graphs is None
    seqs = {f"r{i}": random_tokens(300, V, 100 + i) for i in range(n_req)}
    fed = {r: 0 for r in seqs}

    def both(items):
        outs = []
        for runner in (with_graphs, eager):
            entries = []
            for r, n in items:
                if not runner.has_request(r):
                    runner.add_request(r)
                entries.append(StepEntry(r, list(seqs[r][fed[r]:fed[r] + n]), [n - 1]))
            outs.append(runner.step(entries).float().cpu())
        for r, n in items:
            fed[r] += n
        assert rel_err(outs[0], outs[1]) < TOL[dtype] / 3, (items[0], len(items))
        return outs[0]

    live = list(seqs)
    for i in range(0, n_req, 8):                          # prompts of different lengths, a few a step
        both([(r, 20 + (j * 7) % 40) for j, r in enumerate(live[i:i + 8])])
    before = with_graphs.graphs.replays
    for step in range(12):
        both([(r, 1) for r in live])                      # one bucket, replayed
        if step == 3:                                     # eager work between replays: a portion of a prompt
            both([(live[0], 9)])
        if step == 6:                                     # requests leave: a smaller batch, another bucket
            for r in live[-2:]:
                with_graphs.free_request(r)
                eager.free_request(r)
            live = live[:-2]
    assert with_graphs.graphs.replays - before >= 12
    # a longer context: the next bucket of the context length
    both([(r, 240 if which == "B" else 120) for r in live[:3]])
    for _ in range(3):
        both([(r, 1) for r in live])
    keys = set(with_graphs.graphs.steps)
    assert len(keys) >= 2
    if which == "B":                                      # 70 and 68 requests pad to 80 rows; 512 is the second context bucket
        assert {(80, 256), (80, 512)} <= keys


def test_no_garbage_collection_inside_a_capture(folders):
    """A runner that is dropped is a dead cycle holding captured graphs and their memory. Were it
    collected while the next runner captures a step, its memory would be released in the middle of
    the capture, which ends the process. The capture collects such cycles first and keeps the
    collector off until it is over: here the collector is set to run at every allocation, and the
    forward pass notes whether it is on whenever the stream is capturing."""
    import gc
    dtype, which = "bfloat16", "A"
    V = vocab(which)
    toks = random_tokens(40, V, 77)
    old = gc.get_threshold()
    seen = []

    def decode_some(watch):
        runner = runner_for(folders, which, dtype, max_tokens=256)
        if watch:
            forward = runner.model.forward

            def noting(*a, **k):
                if torch.cuda.is_current_stream_capturing():
                    seen.append(gc.isenabled())
                return forward(*a, **k)
            runner.model.forward = noting
        got = run_plan(runner, {"r": toks}, [[("r", 30)]] + [[("r", 1)]] * 10)["r"]
        assert runner.graphs is not None and runner.graphs.replays >= 10
        return got

    first = decode_some(False)                  # its runner is garbage from here on (a cycle: not freed by counting)
    gc.set_threshold(1, 1, 1)
    try:
        second = decode_some(True)
        assert gc.isenabled()
    finally:
        gc.set_threshold(*old)
    assert seen and not any(seen), "the collector must be off while a step is captured"
    assert torch.equal(first, second)


@pytest.mark.parametrize("which,dtype", [("B", "bfloat16"), ("C", "bfloat16"), ("A", "float32")])
def test_many_decoding_requests_beside_prompt_portions(folders, plain_cache, which, dtype):
    """Ten requests decode while two more are prefilled in portions: in bfloat16 such a step runs the
    decode attention on a second stream beside the prompt attention; both write rows of one output."""
    V = vocab(which)
    seqs = {f"d{i}": random_tokens(30 + 3 * i, V, 500 + i) for i in range(10)}
    seqs["p"] = random_tokens(120, V, 600)
    seqs["q"] = random_tokens(75, V, 601)
    runner = runner_for(folders, which, dtype, max_tokens=64 * 16)
    dec = [r for r in seqs if r.startswith("d")]
    plan = [[(r, len(seqs[r]) - 12) for r in dec]]                          # the decoders' prompts, less 12 tokens
    cuts_p, cuts_q = [40, 33, 5, 30, 12], [20, 2, 41, 12]
    for step in range(12):
        items = [(r, 1) for r in dec]
        if step < len(cuts_p):
            items.append(("p", cuts_p[step]))
        if 2 <= step < 2 + len(cuts_q):
            items.insert(3, ("q", cuts_q[step - 2]))
        plan.append(items)
    assert sum(cuts_p) == 120 and sum(cuts_q) == 75
    got = run_plan(runner, seqs, plan)
    for r, toks in seqs.items():
        assert rel_err(got[r], reference(folders, plain_cache, which, dtype, toks)) < TOL[dtype], r


@pytest.mark.parametrize("stored,run", [("float32", "bfloat16"), ("bfloat16", "float32"), ("float16", "bfloat16"),
                                        ("float16", "float32")])
def test_stored_dtype_differs_from_the_run_dtype(tmp_path, stored, run):
    """A folder stored in one type and run in another: matrices are rounded to bfloat16 for the
    bfloat16 run, widened for the 32-bit run (crates/cuda/src/engine.rs:6572-6598 converts every
    stored type to its run type on the host). The plain implementation takes the stored values."""
    from reinfer_amd.config import config_from_dict
    from reinfer_amd.weights import write_model_folder
    raw, seed = TINY["B"]
    folder = str(tmp_path / f"b_{stored}")
    write_model_folder(config_from_dict(raw), seed, folder, dtype=stored)
    rawr, weights = read_folder(folder)
    toks = random_tokens(90, raw["vocab_size"], 55)
    ref = plain.forward(rawr, weights, toks).float()
    runner = ModelRunner.from_folder(folder, dtype=run, device="cuda:0", max_tokens=128)
    got = run_plan(runner, {"r": toks}, [[("r", 70)], [("r", 2)]] + [[("r", 1)]] * 18)["r"]
    assert rel_err(got, ref) < TOL[run]


@pytest.mark.parametrize("which,dtype", [("B", "float32"), ("C", "bfloat16")])
def test_thousands_of_tokens_of_context(tmp_path, which, dtype):
    """4500 tokens: portions of 2048 with earlier context behind them, then single tokens over a
    context that takes many chunks of the decode kernel and the 8192 bucket of the captured steps."""
    from reinfer_amd.config import config_from_dict
    from reinfer_amd.weights import write_model_folder
    raw = dict(TINY[which][0], max_position_embeddings=8192)
    folder = str(tmp_path / "long")
    write_model_folder(config_from_dict(raw), 3, folder, dtype=dtype)
    rawr, weights = read_folder(folder)
    n = 4500
    toks = random_tokens(n, raw["vocab_size"], 9)
    ref = plain.forward(rawr, weights, toks).float()
    runner = ModelRunner.from_folder(folder, dtype=dtype, device="cuda:0", max_tokens=4544)
    plan = [[("r", 2048)], [("r", 2048)], [("r", 340)]] + [[("r", 1)]] * 64
    got = run_plan(runner, {"r": toks}, plan)["r"]
    assert rel_err(got, ref) < TOL[dtype]
    assert rel_err(got[-64:], ref[-64:]) < TOL[dtype]


@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_short_portions_deep_in_a_long_prompt(tmp_path, which, monkeypatch):
    """Portions of tens to hundreds of tokens behind thousands of cached ones, beside another request's
    from its start: few query tiles with many keys each, which the prompt kernel takes cut by keys, a
    second kernel adding the parts. The steps' plans are watched: tiles cut by keys must have occurred."""
    from reinfer_amd.config import config_from_dict
    from reinfer_amd.weights import write_model_folder
    dtype = "bfloat16"
    raw = dict(TINY[which][0], max_position_embeddings=8192)
    folder = str(tmp_path / "deep")
    write_model_folder(config_from_dict(raw), 21, folder, dtype=dtype)
    rawr, weights = read_folder(folder)
    seqs = {"r": random_tokens(3400, raw["vocab_size"], 31), "s": random_tokens(900, raw["vocab_size"], 32)}
    plan = [[("r", 2048)], [("r", 100), ("s", 300)], [("r", 40), ("s", 5)], [("r", 700), ("s", 200)],
            [("s", 395), ("r", 70)], [("r", 442)]]
    assert sum(n for st in plan for r, n in st if r == "r") == 3400 and sum(n for st in plan for r, n in st if r == "s") == 900
    ops = kernels.current()
    seen = {"cut": 0, "other": 0}
    inner = ops.attention_prefill

    def watched(q, q_stride, out, kc, vc, batch, Hq, Hkv, d, scale, window, group, tiles, n_tiles, ranges=None,
                merge=None, n_merge=0, n_slots=0):
        seen["cut" if n_slots else "other"] += 1
        return inner(q, q_stride, out, kc, vc, batch, Hq, Hkv, d, scale, window, group, tiles, n_tiles, ranges,
                     merge, n_merge, n_slots)
    monkeypatch.setattr(ops, "attention_prefill", watched)
    runner = ModelRunner.from_folder(folder, dtype=dtype, device="cuda:0", max_tokens=4352)
    got = run_plan(runner, seqs, plan)
    assert seen["cut"] > 0
    for r, toks in seqs.items():
        ref = plain.forward(rawr, weights, toks).float()
        assert rel_err(got[r], ref) < TOL[dtype], r
        for lo in (2048, 2148, 2188, 2888, 2958):           # the first token of each deep portion, and its last
            if r == "r":
                assert rel_err(got[r][lo:lo + 1], ref[lo:lo + 1]) < TOL[dtype]
                assert rel_err(got[r][lo - 1:lo], ref[lo - 1:lo]) < TOL[dtype]


@pytest.mark.parametrize("limit,n", [(300, 299), (100, 99)])
def test_context_limit_that_is_no_power_of_two(folders, plain_cache, limit, n):
    """Captured decode steps pad the context to buckets (powers of two from 256); the last bucket is the
    context limit itself, which the block tables are made for: 300 (contexts above 256 once asked for a
    bucket of 512 that the tables did not hold) and 100 (below the smallest bucket)."""
    which, dtype = "B", "bfloat16"
    runner = runner_for(folders, which, dtype, max_tokens=320, max_model_len=limit)
    toks = random_tokens(n, vocab(which), 88)
    first = n - 60
    got = run_plan(runner, {"r": toks}, [[("r", first)]] + [[("r", 1)]] * 60)["r"]
    assert runner.graphs is not None and runner.graphs.replays >= 60
    assert rel_err(got, reference(folders, plain_cache, which, dtype, toks)) < TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_more_requests_than_a_captured_step_holds(folders, plain_cache, dtype):
    """136 requests decode together: above the largest captured batch, so the step runs kernel by kernel
    with the prompt-sized products. Seventeen distinct sequences, each eight times: all agree with the
    plain logits, and twins in one batch with each other."""
    which = "B"
    V = vocab(which)
    distinct = [random_tokens(20 + 2 * i, V, 900 + i) for i in range(17)]
    runner = runner_for(folders, which, dtype, max_tokens=136 * 64, max_seqs=136)
    rids = [f"r{j}" for j in range(136)]
    steps = 5
    for lo in range(0, 136, 17):
        runner_entries = []
        for j in range(lo, lo + 17):
            runner.add_request(rids[j])
            s = distinct[j % 17]
            runner_entries.append(StepEntry(rids[j], s[:len(s) - steps], []))
        runner.step(runner_entries)
    rows = {r: [] for r in rids}
    for k in range(steps):
        out = runner.step([StepEntry(r, [distinct[j % 17][len(distinct[j % 17]) - steps + k]], [0])
                           for j, r in enumerate(rids)]).float().cpu()
        for j, r in enumerate(rids):
            rows[r].append(out[j])
    assert runner.graphs is None or runner.graphs.replays == 0, "136 rows are more than a captured step holds"
    for j, r in enumerate(rids):
        s = distinct[j % 17]
        got = torch.stack(rows[r])
        assert rel_err(got, reference(folders, plain_cache, which, dtype, s)[-steps:]) < TOL[dtype], r
        if j >= 17:
            assert rel_err(got, torch.stack(rows[rids[j % 17]])) < 1e-6, r
        runner.free_request(r)
    runner.manager.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sixteen_thousand_tokens_of_context(tmp_path, dtype):
    """A context of 16,400 tokens: eight portions of 2,048 behind ever longer context, then single tokens
    over more than a thousand blocks (split-KV decode with as many chunks as the chip takes, the 32768
    bucket of the captured steps). The head norms of the first layer are sharpened so that single far
    keys carry weight. The plain side runs in float32 here (a score matrix of 16,400 squared a head)."""
    from reinfer_amd.config import config_from_dict
    from reinfer_amd.weights import write_model_folder
    raw = dict(TINY["A"][0], max_position_embeddings=16500)
    folder = str(tmp_path / "long16k")
    write_model_folder(config_from_dict(raw), 12, folder, dtype=dtype)
    rawr, weights = read_folder(folder)
    weights = {k: v.clone() for k, v in weights.items()}
    for name in ("q_norm", "k_norm"):
        weights[f"model.layers.0.self_attn.{name}.weight"] *= 2.5
    n = 16400
    toks = random_tokens(n, raw["vocab_size"], 13)
    rows = [0, 1, 2047, 2048, 8191, 8192, 12000, 16383] + list(range(16384, n))
    ref = plain.forward(rawr, weights, toks, torch.float32, rows=rows).float()
    runner = ModelRunner.from_config(config_from_dict(raw), dtype=dtype, weights=weights, max_tokens=16448)
    runner.add_request("r")
    got = []
    for lo in range(0, 16384, 2048):
        want = [p - lo for p in rows if lo <= p < lo + 2048]
        out = runner.step([StepEntry("r", toks[lo:lo + 2048], want)])
        if want:
            got.append(out.float().cpu())
    for p in range(16384, n):
        got.append(runner.step([StepEntry("r", [toks[p]], [0])]).float().cpu())
    got = torch.cat(got)
    assert rel_err(got, ref) < TOL[dtype]
    assert rel_err(got[-16:], ref[-16:]) < TOL[dtype]
