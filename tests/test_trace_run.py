"""bin/trace_run as a user runs it: a subprocess fed JSON steps on standard input, answering
``done <step>`` after each and leaving ``<step>.f32`` files, compared with the plain implementation."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_qwen3 as plain
from helpers import TOL, make_folder, random_tokens, read_folder, rel_err

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_mixed_steps(tmp_path, dtype):
    folder = make_folder(tmp_path, "B", "bfloat16")
    raw, weights = read_folder(folder)
    V = raw["vocab_size"]
    seqs = {"a": random_tokens(70, V, 1), "b": random_tokens(41, V, 2), "c": random_tokens(50, V, 3)}
    refs = {r: plain.forward(raw, weights, t) for r, t in seqs.items()}
    # portions beside single tokens; c starts after a has ended, on a's blocks (192 tokens of cache)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": seqs["a"][:33], "want": [0, 32]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": seqs["a"][33:69], "want": list(range(36))},
                                {"id": "b", "tokens": seqs["b"][:2], "want": []}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": seqs["b"][2:40], "want": [37]},
                                {"id": "a", "tokens": seqs["a"][69:70], "want": [0]}], "end": ["a"]},
        {"step": 3, "entries": [{"id": "c", "tokens": seqs["c"][:49], "want": []},
                                {"id": "b", "tokens": seqs["b"][40:41], "want": [0]}], "end": ["b"]},
        {"step": 4, "entries": [{"id": "c", "tokens": seqs["c"][49:50], "want": [0]}], "end": ["c"]},
    ]
    out = tmp_path / f"out_{dtype}"
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
         "--out", str(out), "--max-tokens", "192"],
        input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(5)]
    fed = {r: 0 for r in seqs}
    for s in steps:
        want_rows = []
        for e in s["entries"]:
            want_rows += [refs[e["id"]][fed[e["id"]] + w] for w in e["want"]]
            fed[e["id"]] += len(e["tokens"])
        path = out / f"{s['step']}.f32"
        if not want_rows:
            assert not path.exists()
            continue
        got = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(len(want_rows), V))
        assert rel_err(got, torch.stack(want_rows)) < TOL[dtype]


@pytest.mark.parametrize("which,dtype", [("C", "float32"), ("B", "bfloat16")])
def test_trace_run_orders_ids_and_idle_requests(tmp_path, which, dtype):
    """What a trace may do beside the plain cases: ``want`` in any order and with a place twice, an
    entry of a decode step that wants nothing, a step in which nothing is wanted at all (no file), a
    request left out of steps and going on later, a request that ends while idle, an id that is a
    number, and an id used again after its end (a fresh request on used blocks)."""
    folder = make_folder(tmp_path, which, dtype)
    raw, weights = read_folder(folder)
    V = raw["vocab_size"]
    a, b, c, a2 = (random_tokens(n, V, s) for n, s in ((40, 1), (30, 2), (20, 3), (25, 4)))
    ra, rb, ra2 = (plain.forward(raw, weights, t).float() for t in (a, b, a2))
    steps = [
        ({"step": 0, "entries": [{"id": "a", "tokens": a[:10], "want": [9, 0, 3]},
                                 {"id": 7, "tokens": b[:2], "want": []}], "end": []}, ra[[9, 0, 3]]),
        ({"step": 1, "entries": [{"id": "a", "tokens": a[10:11], "want": []},
                                 {"id": 7, "tokens": b[2:3], "want": [0]}], "end": []}, rb[[2]]),
        ({"step": 2, "entries": [{"id": 7, "tokens": b[3:30], "want": [26, 26, 0]}], "end": []}, rb[[29, 29, 3]]),
        ({"step": 3, "entries": [{"id": "c", "tokens": c, "want": []}], "end": [7]}, None),
        ({"step": 4, "entries": [{"id": "a", "tokens": a[11:40], "want": [28]}], "end": ["a", "c"]}, ra[[39]]),
        ({"step": 5, "entries": [{"id": "a", "tokens": a2[:24], "want": [23]}], "end": []}, ra2[[23]]),
        ({"step": 6, "entries": [{"id": "a", "tokens": a2[24:25], "want": [0]}], "end": ["a"]}, ra2[[24]]),
    ]
    out = tmp_path / "out"
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
         "--out", str(out), "--max-tokens", "192"],
        input="".join(json.dumps(s) + "\n" for s, _ in steps), capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(7)]
    for s, ref in steps:
        path = out / f"{s['step']}.f32"
        if ref is None:
            assert not path.exists()
            continue
        got = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(ref.shape[0], V))
        assert rel_err(got, ref) < TOL[dtype], s["step"]


def test_trace_run_step_by_step_over_a_pipe(tmp_path):
    """The caller writes one step, waits for ``done <step>``, then writes the next: every answer comes
    without further input, the step's file is whole when the answer is printed, and the end of the
    input ends the program with status 0."""
    folder = make_folder(tmp_path, "A", "bfloat16")
    raw, weights = read_folder(folder)
    toks = random_tokens(24, raw["vocab_size"], 5)
    ref = plain.forward(raw, weights, toks).float()
    out = tmp_path / "out"
    proc = subprocess.Popen(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "bfloat16",
         "--out", str(out), "--max-tokens", "64"],
        stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, bufsize=1)
    try:
        fed = 0
        for step in range(13):
            n = 12 if step == 0 else 1
            rec = {"step": step, "entries": [{"id": "a", "tokens": toks[fed:fed + n], "want": [n - 1]}], "end": []}
            proc.stdin.write(json.dumps(rec) + "\n")
            proc.stdin.flush()
            assert proc.stdout.readline().strip() == f"done {step}"
            fed += n
            got = torch.from_numpy(np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(1, -1))
            assert rel_err(got, ref[fed - 1:fed]) < TOL["bfloat16"]
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0
    finally:
        if proc.poll() is None:
            proc.kill()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_dumps_the_hidden_state_behind_every_layer(tmp_path, dtype):
    """``--dump-layer``: a step's file holds the hidden state of its tokens behind the embedding and behind
    every layer, in the order of the entries; against the plain implementation's, layer by layer, for a
    portion of a prompt behind earlier context beside a single decoded token."""
    folder = make_folder(tmp_path, "C", "bfloat16")
    raw, weights = read_folder(folder)
    V, h, L = raw["vocab_size"], raw["hidden_size"], raw["num_hidden_layers"]
    seqs = {"a": random_tokens(45, V, 4), "b": random_tokens(30, V, 5)}
    hid = {r: torch.stack(plain.hidden_states(raw, weights, t)) for r, t in seqs.items()}      # [L + 1, T, h]
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": seqs["a"][:20], "want": []},
                                {"id": "b", "tokens": seqs["b"][:29], "want": []}], "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": seqs["b"][29:30], "want": [0]},
                                {"id": "a", "tokens": seqs["a"][20:45], "want": [24]}], "end": ["a", "b"]},
    ]
    out, dump = tmp_path / f"out_{dtype}", tmp_path / f"layers_{dtype}"
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
         "--out", str(out), "--max-tokens", "128", "--dump-layer", str(dump)],
        input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    got0 = torch.from_numpy(np.fromfile(dump / "0.layers.f32", dtype="<f4").reshape(L + 1, 49, h))
    got1 = torch.from_numpy(np.fromfile(dump / "1.layers.f32", dtype="<f4").reshape(L + 1, 26, h))
    want0 = torch.cat([hid["a"][:, :20], hid["b"][:, :29]], dim=1)
    want1 = torch.cat([hid["b"][:, 29:30], hid["a"][:, 20:45]], dim=1)
    assert torch.equal(got0[0], want0[0].float()), "the embedding rows are copies"
    for layer in range(1, L + 1):
        assert rel_err(got0[layer], want0[layer]) < TOL[dtype], layer
        assert rel_err(got1[layer], want1[layer]) < TOL[dtype], layer
    # the logits files are what they are without the option
    assert (out / "1.f32").exists() and not (out / "0.f32").exists()


def test_trace_run_checks_start_against_what_the_cache_holds(tmp_path):
    """An entry may say where it starts. A right ``start`` changes nothing; a trace that skips tokens (or
    repeats them, or starts a fresh request elsewhere than at 0) ends the replay with status 4 before that
    step runs: the steps before it are answered, the bad one is not and leaves no file."""
    folder = make_folder(tmp_path, "A", "float32")
    raw, weights = read_folder(folder)
    V = raw["vocab_size"]
    a, b = random_tokens(20, V, 8), random_tokens(9, V, 9)
    ref = plain.forward(raw, weights, a).float()

    def run(steps, name):
        out = tmp_path / name
        proc = subprocess.run(
            [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
             "--out", str(out), "--max-tokens", "128"],
            input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
        return proc, out

    good = [
        {"step": 0, "entries": [{"id": "a", "start": 0, "tokens": a[:12], "want": [11]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "start": 12, "tokens": a[12:20], "want": [7]},
                                {"id": "b", "tokens": b, "want": []}], "end": ["a"]},
        # the id again after its end: a fresh request, which starts at 0
        {"step": 2, "entries": [{"id": "a", "start": 0, "tokens": a[:3], "want": [2]},
                                {"id": "b", "start": 9, "tokens": [1], "want": []}], "end": []},
    ]
    proc, out = run(good, "good")
    assert proc.returncode == 0, proc.stderr[-2000:]
    got = torch.from_numpy(np.fromfile(out / "1.f32", dtype="<f4").reshape(1, V))
    assert rel_err(got, ref[19:20]) < TOL["float32"]

    for name, bad in (("skips", {"id": "a", "start": 14, "tokens": a[14:20], "want": [5]}),
                      ("repeats", {"id": "a", "start": 10, "tokens": a[10:20], "want": [9]}),
                      ("fresh", {"id": "z", "start": 5, "tokens": a[5:9], "want": [3]})):
        steps = [good[0], {"step": 1, "entries": [{"id": "b", "tokens": b, "want": [0]}, bad], "end": []}]
        proc, out = run(steps, name)
        assert proc.returncode == 4, (name, proc.returncode, proc.stderr[-2000:])
        assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == ["done 0"]
        assert (out / "0.f32").exists() and not (out / "1.f32").exists()
        assert "start" in proc.stderr and repr(bad["id"]) in proc.stderr
