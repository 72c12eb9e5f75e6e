"""Configurations and cut plans drawn at random (fixed seeds): head sizes in steps of 16 up to 256, any
number of heads and groups, widths and vocabularies that are no power of two, windows on some layers,
tied and separate heads; up to four live requests, portions beside single tokens, requests left out
of steps, a cache with room for exactly the four largest. Both dtypes against the plain implementation;
everything a request does not own is NaN."""
import random

import pytest
import torch

import plain_qwen3 as plain
from helpers import TOL, random_tokens, read_folder, rel_err, run_plan
from reinfer_amd.config import config_from_dict
from reinfer_amd.engine import ModelRunner
from reinfer_amd.weights import write_model_folder

pytestmark = pytest.mark.gpu


def draw_config(rng):
    kv, g, layers = rng.choice([1, 2, 3, 4, 5, 8]), rng.choice([1, 2, 3, 4, 6, 7, 8]), rng.choice([1, 2, 3])
    raw = {"architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "num_hidden_layers": layers,
           "hidden_size": rng.choice([72, 200, 264, 328, 520, 1000, 1024]),
           "num_attention_heads": kv * g, "num_key_value_heads": kv,
           "head_dim": rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 256]),
           "intermediate_size": rng.choice([88, 176, 456, 1000, 1368]), "vocab_size": rng.choice([333, 1003, 5001]),
           "rope_theta": rng.choice([10000.0, 1e6, 5e4]), "rms_norm_eps": rng.choice([1e-6, 1e-5, 3e-4]),
           "tie_word_embeddings": rng.random() < 0.5, "max_position_embeddings": rng.choice([521, 600, 777, 1000, 1024]),
           "attention_bias": False,
           "hidden_act": "silu", "rope_scaling": None, "sliding_window": None, "use_sliding_window": False}
    if rng.random() < 0.4:
        raw.update(sliding_window=rng.choice([5, 16, 21, 64, 100]), use_sliding_window=True,
                   max_window_layers=rng.randrange(0, layers))
    return raw


def draw_plan(rng, lens):
    """Steps of (request, tokens) with at most four live requests; -> (plan, ends)."""
    fed = {r: 0 for r in lens}
    waiting = list(lens)
    rng.shuffle(waiting)
    live, plan, ends = [], [], {}
    while live or waiting:
        while waiting and len(live) < 4 and (not live or rng.random() < 0.7):
            live.append(waiting.pop(0))
        items = []
        for r in live:
            if len(live) > 1 and rng.random() < 0.2:
                continue                                       # left out of this step
            n = min(lens[r] - fed[r], rng.choice([1, 1, 1, 2, 3, 7, 16, 17, 33, 64, 65, 100, 129, 300]))
            items.append((r, n))
            fed[r] += n
        if not items:
            continue
        plan.append(items)
        done = [r for r in live if fed[r] == lens[r]]
        ends[len(plan) - 1] = done
        live = [r for r in live if r not in done]
    return plan, ends


@pytest.mark.parametrize("seed", [0, 3, 4])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_random_configurations_and_plans(tmp_path, seed, dtype):
    rng = random.Random(seed)
    for ci in range(3):
        raw = draw_config(rng)
        folder = str(tmp_path / f"m{ci}")
        write_model_folder(config_from_dict(raw), 10 * seed + ci, folder, dtype=dtype)
        rawr, weights = read_folder(folder)
        lens = {r: rng.choice([3, 40, 97, 130, 200, 333, 520]) for r in "abcde"}
        seqs = {r: random_tokens(n, raw["vocab_size"], 7 * ci + i) for i, (r, n) in enumerate(lens.items())}
        plan, ends = draw_plan(rng, lens)
        room = sum(sorted((n + 63) // 64 * 64 for n in lens.values())[-4:])
        runner = ModelRunner.from_folder(folder, dtype=dtype, device="cuda:0", max_tokens=room)
        for c in runner.caches:
            if c is not None and c.k is not None:
                c.k.fill_(float("nan"))
                c.v.fill_(float("nan"))
        runner.poison_freed_blocks()       # a block that goes back (request ended, window passed) reads NaN from then on
        got = run_plan(runner, seqs, plan, ends=ends)
        assert all(p.num_free == p.num_blocks for p in runner.manager.pools)
        # bfloat16: the bound of helpers.TOL is for three layers; these have at most three
        for r, toks in seqs.items():
            err = rel_err(got[r], plain.forward(rawr, weights, toks).float())
            assert err < TOL[dtype], (seed, ci, r, raw, plan[:8])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", [
    dict(hidden_size=132, intermediate_size=260, head_dim=16, num_attention_heads=9, num_key_value_heads=9, vocab_size=1001),
    dict(hidden_size=100, intermediate_size=90, head_dim=32, num_attention_heads=6, num_key_value_heads=3, vocab_size=257),
    dict(hidden_size=200, intermediate_size=4, head_dim=32, num_attention_heads=2, num_key_value_heads=2, vocab_size=2),
])
def test_sizes_that_the_matrix_core_kernels_do_not_take(tmp_path, sizes, dtype):
    """Widths that are no multiple of 8 (rows are not whole 16-byte pieces), a feed-forward of 4, a
    vocabulary of 2: what the weight-streaming kernels refuse goes to the plain kernels, at every row
    count, with no norm riding on a product that cannot carry it."""
    raw = {"architectures": ["Qwen3ForCausalLM"], "num_hidden_layers": 2, "rope_theta": 10000.0, "rms_norm_eps": 1e-6,
           "tie_word_embeddings": sizes["vocab_size"] % 2 == 1, "max_position_embeddings": 300, **sizes}
    folder = str(tmp_path / "m")
    write_model_folder(config_from_dict(raw), 5, folder, dtype=dtype)
    rawr, weights = read_folder(folder)
    seqs = {r: random_tokens(n, raw["vocab_size"], 9 + i) for i, (r, n) in enumerate((("a", 150), ("b", 70), ("c", 9)))}
    runner = ModelRunner.from_folder(folder, dtype=dtype, device="cuda:0", max_tokens=320)
    plan = [[("a", 100), ("b", 2)], [("a", 1), ("b", 66), ("c", 9)], [("a", 49), ("b", 1)], [("b", 1)]]
    got = run_plan(runner, seqs, plan)
    for r, toks in seqs.items():
        assert rel_err(got[r], plain.forward(rawr, weights, toks).float()) < TOL[dtype], r


def test_head_size_that_is_no_multiple_of_16_is_refused(tmp_path):
    raw = {"architectures": ["Qwen3ForCausalLM"], "num_hidden_layers": 1, "hidden_size": 64, "intermediate_size": 96,
           "head_dim": 24, "num_attention_heads": 4, "num_key_value_heads": 2, "vocab_size": 100,
           "max_position_embeddings": 64}
    folder = str(tmp_path / "m")
    write_model_folder(config_from_dict(raw), 0, folder, dtype="bfloat16")
    with pytest.raises(ValueError, match="steps of 16"):
        ModelRunner.from_folder(folder, dtype="bfloat16", device="cuda:0", max_tokens=64)
