"""The step function's bookkeeping on the CPU: ragged batches, block tables, cache
slots, windows and page reuse, with a stand-in for the kernels, against the plain
implementation. Kernel numerics are the GPU tests' business."""
import pytest
import torch

import plain_qwen3 as plain
from helpers import TINY, make_folder, random_tokens, read_folder, rel_err
from kernel_double import KernelDouble
from reinfer_amd import kernels
from reinfer_amd.cache import OutOfBlocks
from reinfer_amd.engine import ModelRunner, StepEntry, StepError


def build(tmp_path, which, **limits):
    folder = make_folder(tmp_path, which, "float32")
    raw, weights = read_folder(folder)
    runner = ModelRunner.from_folder(folder, dtype="float32", device="cpu", **limits)
    return raw, weights, runner


@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_whole_prompt_matches_plain(tmp_path, which):
    with kernels.use(KernelDouble()):
        raw, weights, runner = build(tmp_path, which, max_tokens=128)
        toks = random_tokens(45, raw["vocab_size"], 7)
        ref = plain.forward(raw, weights, toks)
        runner.add_request("a")
        got = runner.step([StepEntry("a", toks, list(range(len(toks))))])
        assert rel_err(got, ref) < 2e-5
        runner.free_request("a")
        runner.manager.check()


@pytest.mark.parametrize("which", ["A", "C"])
def test_portions_and_decode_match_whole(tmp_path, which):
    with kernels.use(KernelDouble()):
        raw, weights, runner = build(tmp_path, which, max_tokens=128)
        toks = random_tokens(61, raw["vocab_size"], 11)
        ref = plain.forward(raw, weights, toks)
        runner.add_request("a")
        cuts = [7, 2, 16, 3, 2, 17, 2]          # then one by one
        rows, pos = [], 0
        for c in cuts:
            rows.append(runner.step([StepEntry("a", toks[pos:pos + c], list(range(c)))]))
            pos += c
        while pos < len(toks):
            rows.append(runner.step([StepEntry("a", toks[pos:pos + 1], [0])]))
            pos += 1
        assert rel_err(torch.cat(rows), ref) < 2e-5


def test_mixed_batch_with_reuse(tmp_path):
    """Four requests, portions beside decoded tokens, so few blocks that they are used again."""
    with kernels.use(KernelDouble()):
        raw, weights, runner = build(tmp_path, "C", max_tokens=160, block_size=16)
        V = raw["vocab_size"]
        seqs = {r: random_tokens(n, V, 100 + i) for i, (r, n) in enumerate([("a", 40), ("b", 33), ("c", 50), ("d", 29), ("e", 47)])}
        refs = {r: plain.forward(raw, weights, t) for r, t in seqs.items()}
        got = {r: [] for r in seqs}
        fed = {r: 0 for r in seqs}
        # a, b start; c joins; a ends -> its blocks go to d; e takes b's
        plan = [
            [("a", 9), ("b", 2)],
            [("a", 1), ("b", 20), ("c", 5)],
            [("a", 30), ("b", 1), ("c", 1)],
            [("b", 10), ("c", 44)],             # a finished after step 2
            [("d", 29), ("e", 3)],
            [("e", 44)],
        ]
        ends = {2: ["a"], 3: ["b", "c"], 4: ["d"], 5: ["e"]}
        for step, items in enumerate(plan):
            entries = []
            for r, n in items:
                if not runner.has_request(r):
                    runner.add_request(r)
                entries.append(StepEntry(r, seqs[r][fed[r]:fed[r] + n], list(range(n))))
            out = runner.step(entries)
            o = 0
            for r, n in items:
                got[r].append(out[o:o + n])
                o += n
                fed[r] += n
            for r in ends.get(step, []):
                runner.free_request(r)
            runner.manager.check()
        for r in seqs:
            assert fed[r] == len(seqs[r])
            assert rel_err(torch.cat(got[r]), refs[r]) < 2e-5, r
        assert runner.manager.pools[0].allocs > runner.manager.pools[0].num_blocks   # blocks were used again
        assert all(p.num_free == p.num_blocks for p in runner.manager.pools)


def test_step_errors(tmp_path):
    with kernels.use(KernelDouble()):
        raw, weights, runner = build(tmp_path, "A", max_tokens=64)
        runner.add_request("a")
        with pytest.raises(StepError, match="vocabulary"):
            runner.step([StepEntry("a", [raw["vocab_size"]], [0])])
        with pytest.raises(StepError, match="no tokens"):
            runner.step([StepEntry("a", [], [])])
        with pytest.raises(StepError, match="not live"):
            runner.step([StepEntry("zz", [1], [0])])
        with pytest.raises(StepError, match="twice"):
            runner.step([StepEntry("a", [1], [0]), StepEntry("a", [2], [0])])
        with pytest.raises(StepError, match="wanted"):
            runner.step([StepEntry("a", [1, 2], [2])])
        with pytest.raises(OutOfBlocks):
            runner.step([StepEntry("a", [1] * 65, [0])])
        # a refused step leaves nothing behind
        assert runner.num_tokens("a") == 0
        assert all(p.num_free == p.num_blocks for p in runner.manager.pools)
        with pytest.raises(StepError, match="context"):
            runner2 = ModelRunner.from_folder(make_folder(tmp_path, "A", "float32"), dtype="float32",
                                              device="cpu", max_tokens=1024)
            runner2.add_request("x")
            runner2.step([StepEntry("x", [1] * 257, [0])])


def test_no_logits_wanted_still_stores(tmp_path):
    with kernels.use(KernelDouble()):
        raw, weights, runner = build(tmp_path, "B", max_tokens=64)
        toks = random_tokens(20, raw["vocab_size"], 3)
        ref = plain.forward(raw, weights, toks)
        runner.add_request("a")
        out = runner.step([StepEntry("a", toks[:19], [])])
        assert out.shape == (0, raw["vocab_size"])
        got = runner.step([StepEntry("a", toks[19:], [0])])
        assert rel_err(got, ref[19:]) < 2e-5


class CountingDouble(KernelDouble):
    def __init__(self, rows):
        super().__init__()
        self.NORM_ON_PRODUCTS_ROWS = rows
        self.norm_calls = 0

    def add_rmsnorm(self, *a, **k):
        self.norm_calls += 1
        return super().add_rmsnorm(*a, **k)


@pytest.mark.parametrize("which", ["A", "B"])
def test_norm_carried_by_products_equals_norm_kernel(tmp_path, which):
    """bfloat16, few rows: the parts hand the norm between layers to the products around it
    (two norm launches a step remain: before the first layer and before the head). The logits
    agree with the step that launches every norm, and with the plain implementation."""
    folder = make_folder(tmp_path, which, "bfloat16")
    raw, weights = read_folder(folder)
    toks = random_tokens(23, raw["vocab_size"], 5)
    ref = plain.forward(raw, weights, toks)
    L = raw["num_hidden_layers"]
    got = {}
    for rows in (0, 64):
        double = CountingDouble(rows)
        with kernels.use(double):
            runner = ModelRunner.from_folder(folder, dtype="bfloat16", device="cpu", max_tokens=128)
            runner.add_request("a")
            parts = [runner.step([StepEntry("a", toks[:9], list(range(9)))])]
            for i in range(9, len(toks)):
                parts.append(runner.step([StepEntry("a", toks[i:i + 1], [0])]))
            got[rows] = torch.cat(parts)
            steps = 1 + len(toks) - 9
            assert double.norm_calls == steps * ((2 * L + 1) if rows == 0 else 2)
    assert rel_err(got[64], got[0]) < 2e-2
    assert rel_err(got[64], ref) < 3e-2 and rel_err(got[0], ref) < 3e-2
