"""The line that bench.py prints: its keys and the figures' consistency, on two layers of the default shape."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_line_holds_the_contract():
    """A test of the line's format: its keys, the flat configuration and the arithmetic between its figures. It
    says nothing about whether the timed work is the model's (a bench that skipped work would pass it); that is
    what the parity tests at these widths and ``check_run`` below are for."""
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--layers", "2", "--steps", "8", "--warmup", "4",
                        "--no-points", "--profile-steps", "1"], capture_output=True, text=True, timeout=600, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [ln for ln in r.stdout.splitlines() if ln.startswith("{")]
    assert len(lines) == 1, "one JSON line on standard output"
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 8 and d["warmup"] == 4 and d["higher_is_better"] is True
    assert d["dtype"] == "bf16" and "synthetic" in d["data"] and d["unit"] == "tok/s"
    cfg = d["config"]
    assert len(cfg) <= 20 and all(not isinstance(v, (dict, list)) for v in cfg.values()), "flat, at most 20 keys"
    assert cfg["layers"] == 2 and cfg["layers_of_model"] == 36 and cfg["global_batch"] == 8
    assert cfg["hidden"] == 4096 and cfg["intermediate"] == 12288 and cfg["vocab"] == 151936
    # value is decoded tokens a second of the timed steps
    assert abs(d["value"] - cfg["global_batch"] / (d["ms_per_step"] * 1e-3)) <= 0.01 * d["value"]
    p = d["prefill"]
    assert set(p) >= {"value", "tokens", "ms", "frac"} and p["tokens"] == 2048
    assert abs(p["value"] - p["tokens"] / (p["ms"] * 1e-3)) <= 0.01 * p["value"] and 0 < p["frac"] < 1
    rf = d["roofline"]
    assert rf["bound"] == "hbm" and rf["unit"] == "GB/s" and rf["peak"] == 8000.0
    assert abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-3 and 0 < rf["frac"] < 1
    assert "kernel_ms" in d and d["kernel_ms"]["attention"]["ms"] > 0


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120, cwd=ROOT)
    assert r.returncode == 2 and "one GPU" in (r.stdout + r.stderr)


def test_bench_refuses_a_run_whose_results_are_not_a_models():
    """``bench.check_run`` stands between every timed run and the line: logits that are not all finite, or a
    request without tokens of the vocabulary, raise and nothing is printed."""
    import torch
    sys.path.insert(0, ROOT)
    import bench
    from helpers import TINY_A
    from reinfer_amd.config import config_from_dict
    from reinfer_amd.engine import LLMEngine
    from reinfer_amd.sampling import SamplingParams
    eng = LLMEngine(config=config_from_dict(TINY_A), seed=0, dtype="bfloat16", num_blocks=32)
    for p in ([1, 2, 3, 4, 5], [7, 8, 9]):
        eng.add_request(p, SamplingParams(temperature=0.0, max_tokens=50, ignore_eos=True))
    for _ in range(4):
        eng.step()
    running = list(eng.scheduler.running)
    bench.check_run(eng, TINY_A, running, "a good run")
    eng.runner.last_logits[1, 17] = float("nan")
    with pytest.raises(bench.InvalidRun, match="finite"):
        bench.check_run(eng, TINY_A, running, "a bad run")
    eng.step()
    bench.check_run(eng, TINY_A, running, "the next step's logits are whole again")
    with pytest.raises(bench.InvalidRun, match="vocabulary"):
        bench.check_run(eng, dict(TINY_A, vocab_size=1), running, "tokens outside a vocabulary of one")
