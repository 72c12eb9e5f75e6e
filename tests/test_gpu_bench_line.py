"""The line that bench.py prints: its keys and the figures' consistency, on two layers of the default shape."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_line_holds_the_contract():
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
