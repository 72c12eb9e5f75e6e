"""The serving kernels at the sizes they are built for, against the plain implementation.

Models with the widths of the Qwen3-8B shape (4096 wide, 32 query heads over 8 KV heads of 128,
feed-forward 12288, vocabulary 151936; two layers), of the Qwen3-4B shape (2560 wide with a 4096-wide
q projection, tied head; one layer) and of the Qwen3-32B shape (5120 wide, 64 query heads in groups
of 8, feed-forward 25600; one layer), random weights. The reference is ``plain_qwen3.forward`` in
float32 on the CPU with the very same tensors (drawn once, on the GPU, and copied; the generator
gives the same values on either device), at the wanted positions only. Both precisions of the
engine are compared with it under the ways of cutting the work that the product runs at these widths:
whole prompts, the last tokens one by one, portions of changing size, requests mixed in one step, a
2,048-token prompt in one step and in portions behind earlier context, and 17, 33 and 64 requests
decoding together (the products over K ranges, the captured steps), metric and bounds as for the
tiny models (crates/cuda/tests/parity.rs:22-27)."""
import pytest
import torch

import plain_qwen3 as plain
from helpers import TOL, random_tokens, rel_err
from reinfer_amd import kernels
from reinfer_amd.config import config_from_dict
from reinfer_amd.engine import ModelRunner, StepEntry
from reinfer_amd.models import declare_params
from reinfer_amd.weights import random_tensors

pytestmark = pytest.mark.gpu


def raw_config(layers, hidden, heads, inter, tied):
    return {"architectures": ["Qwen3ForCausalLM"], "num_hidden_layers": layers, "hidden_size": hidden,
            "num_attention_heads": heads, "num_key_value_heads": 8, "head_dim": 128, "intermediate_size": inter,
            "vocab_size": 151936, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": tied,
            "max_position_embeddings": 4096}


SHAPES = {"8b": raw_config(2, 4096, 32, 12288, False), "4b": raw_config(1, 2560, 32, 9728, True),
          "32b": raw_config(1, 5120, 64, 25600, False)}


class Width:
    """One shape: the weights, a runner per precision, and the plain logits of sequences by name."""

    def __init__(self, name: str, max_tokens: int, max_seqs: int):
        assert kernels.current().name == "hip-gfx950"
        self.raw = SHAPES[name]
        cfg = config_from_dict(self.raw)
        dev = torch.device("cuda:0")
        weights = random_tensors(declare_params(cfg.to_spec()), 7, torch.bfloat16, dev)
        self.cpu = {k: v.float().cpu() for k, v in weights.items()}
        self.runners = {dt: ModelRunner.from_config(cfg, dtype=dt, device="cuda:0", weights=weights,
                                                    max_tokens=max_tokens, max_seqs=max_seqs)
                        for dt in ("float32", "bfloat16")}
        self.seqs = {}
        self._plain = {}

    def seq(self, key: str, n: int, seed: int):
        self.seqs.setdefault(key, random_tokens(n, self.raw["vocab_size"], seed))
        return self.seqs[key]

    def plain_rows(self, key: str, rows):
        """Plain float32 logits of sequence ``key`` at ``rows``; a sequence's rows are computed once."""
        rows = tuple(rows)
        if (key, rows) not in self._plain:
            self._plain[(key, rows)] = plain.forward(self.raw, self.cpu, self.seqs[key], torch.float32, rows=rows)
        return self._plain[(key, rows)]


@pytest.fixture(scope="module")
def w8():
    w = Width("8b", max_tokens=100 * 384, max_seqs=100)
    yield w
    del w
    torch.cuda.empty_cache()


def feed(runner, seqs, plan, wanted):
    """plan: steps of (request, n tokens). ``wanted[r]`` = positions of r whose logits are compared.
    -> {r: logits at wanted[r], in order}"""
    got = {r: {} for r in seqs}
    fed = {r: 0 for r in seqs}
    for items in plan:
        entries, marks = [], []
        for r, n in items:
            if not runner.has_request(r):
                runner.add_request(r)
            want = [p - fed[r] for p in wanted[r] if fed[r] <= p < fed[r] + n]
            entries.append(StepEntry(r, seqs[r][fed[r]:fed[r] + n], want))
            marks.append((r, [p for p in wanted[r] if fed[r] <= p < fed[r] + n]))
            fed[r] += n
        out = runner.step(entries).float().cpu()
        o = 0
        for r, ps in marks:
            for p in ps:
                got[r][p] = out[o]
                o += 1
        assert o == out.shape[0]
        for r, _ in items:
            if fed[r] == len(seqs[r]):
                runner.free_request(r)
        runner.manager.check()
    return {r: torch.stack([got[r][p] for p in wanted[r]]) for r in seqs}


def check(w, dtype, seqs, plan, wanted):
    got = feed(w.runners[dtype], seqs, plan, wanted)
    for r in seqs:
        ref = w.plain_rows(r, wanted[r])
        err = rel_err(got[r], ref)
        assert err < TOL[dtype], (r, dtype, err)


def every(n, step):
    return sorted(set(range(0, n, step)) | {n - 1})


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_four_cuts_at_the_8b_widths(w8, dtype):
    seqs = {"a": w8.seq("a", 150, 1), "b": w8.seq("b", 97, 2), "c": w8.seq("c", 40, 3)}
    wanted = {"a": every(150, 7), "b": every(97, 5), "c": list(range(40))}
    # whole
    check(w8, dtype, seqs, [[("a", 150)], [("b", 97)], [("c", 40)]], wanted)
    # most in one step, the last 32 one by one
    one_by_one = []
    for r, n in (("a", 150), ("b", 97), ("c", 40)):
        one_by_one += [[(r, n - 32)]] + [[(r, 1)]] * 32
    check(w8, dtype, seqs, one_by_one, {r: [p for p in wanted[r] if p >= len(seqs[r]) - 40] for r in seqs})
    # portions of changing size, down to two tokens
    check(w8, dtype, seqs, [[("a", 2)], [("a", 61)], [("a", 3)], [("a", 80)], [("a", 4)],
                            [("b", 33)], [("b", 2)], [("b", 62)], [("c", 17)], [("c", 2)], [("c", 21)]], wanted)
    # mixed: portions of some beside single tokens of others; blocks of finished requests are used again
    mixed = [[("a", 70), ("b", 2)], [("a", 1), ("b", 60), ("c", 17)], [("a", 65), ("b", 1), ("c", 1)],
             [("a", 1), ("b", 34), ("c", 2)]] + [[("a", 1), ("c", 1)]] * 13 + [[("c", 7)]]
    check(w8, dtype, seqs, mixed, wanted)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_2048_token_prompt_whole_and_in_portions(w8, dtype):
    """The prompt kernels at the length the bench runs them: one step of 2,048 tokens, and four portions
    of 512 behind 300 tokens of earlier context (query tiles listed twice, keys from the cache)."""
    n = 2348
    seqs = {"long": w8.seq("long", n, 11)}
    wanted = {"long": sorted({0, 1, 15, 16, 17, 299, 300, 301, 811, 812, 1023, 1024, 1323, 1324, 1836, 2047, 2048,
                              2300, n - 2, n - 1})}
    check(w8, dtype, seqs, [[("long", 2048)], [("long", n - 2048)]], wanted)
    check(w8, dtype, seqs, [[("long", 300)]] + [[("long", 512)]] * 4, wanted)


@pytest.mark.parametrize("n_req", [17, 33, 64, 100])
def test_many_requests_decode_together_at_the_8b_widths(w8, n_req):
    """The decode step the bench times: 17, 33, 64 and 100 requests, each with a context of 300 and more tokens,
    decode together for 10 steps (bfloat16: products over K ranges whose sums the next kernel adds, the
    q/k norm on those sums, flash decode at that batch, captured steps; above 64 rows the library's products
    beside the down projection over K ranges). Eight distinct sequences are
    repeated over the requests: twins must agree to the bit, and all with the plain logits."""
    distinct = {f"s{i}": w8.seq(f"s{i}", 300 + 3 * i + 10, 20 + i) for i in range(8)}
    steps = 10
    for dtype in ("bfloat16", "float32"):
        if dtype == "float32" and n_req != 33:
            continue                                   # one batch size is enough for the 32-bit path
        runner = w8.runners[dtype]
        rids = [f"r{j}" for j in range(n_req)]
        src = {r: f"s{j % 8}" for j, r in enumerate(rids)}
        for r in rids:
            runner.add_request(r)
        # prompts, eight requests a step
        for lo in range(0, n_req, 8):
            entries = [StepEntry(r, distinct[src[r]][:len(distinct[src[r]]) - steps], []) for r in rids[lo:lo + 8]]
            runner.step(entries)
        rows = {r: [] for r in rids}
        for k in range(steps):
            entries = []
            for r in rids:
                s = distinct[src[r]]
                entries.append(StepEntry(r, [s[len(s) - steps + k]], [0]))
            out = runner.step(entries).float().cpu()
            for j, r in enumerate(rids):
                rows[r].append(out[j])
        for r in rids:
            runner.free_request(r)
        runner.manager.check()
        for j, r in enumerate(rids):
            s = distinct[src[r]]
            got = torch.stack(rows[r])
            ref = w8.plain_rows(src[r], range(len(s) - steps, len(s)))
            err = rel_err(got, ref)
            assert err < TOL[dtype], (r, dtype, n_req, err)
            if j >= 8:
                assert torch.equal(got, torch.stack(rows[rids[j % 8]])), (r, "differs from its twin in the same batch")


@pytest.mark.parametrize("shape", ["4b", "32b"])
def test_other_full_widths(shape):
    """One layer of the Qwen3-4B widths (q projection wider than the model, tied head, K = 2560 and 9728: no
    multiple of the products' 1024-wide walk) and of the Qwen3-32B widths (groups of 8 query heads,
    feed-forward 25600): prompts whole and in portions, then 1, 8 and 20 requests decoding together."""
    w = Width(shape, max_tokens=24 * 256, max_seqs=24)
    try:
        seqs = {"a": w.seq("a", 131, 1), "b": w.seq("b", 70, 2)}
        wanted = {"a": every(131, 9), "b": every(70, 6)}
        for dtype in ("float32", "bfloat16"):
            check(w, dtype, seqs, [[("a", 131)], [("b", 70)]], wanted)
            check(w, dtype, seqs, [[("a", 40), ("b", 3)], [("a", 1), ("b", 60)], [("a", 88), ("b", 1)],
                                   [("a", 2), ("b", 6)]], wanted)
        distinct = {f"s{i}": w.seq(f"s{i}", 90 + 5 * i, 30 + i) for i in range(4)}
        steps = 6
        for n_req in (1, 8, 20):
            runner = w.runners["bfloat16"]
            rids = [f"r{j}" for j in range(n_req)]
            src = {r: f"s{j % 4}" for j, r in enumerate(rids)}
            for r in rids:
                runner.add_request(r)
            for lo in range(0, n_req, 8):
                runner.step([StepEntry(r, distinct[src[r]][:len(distinct[src[r]]) - steps], []) for r in rids[lo:lo + 8]])
            rows = {r: [] for r in rids}
            for k in range(steps):
                out = runner.step([StepEntry(r, [distinct[src[r]][len(distinct[src[r]]) - steps + k]], [0])
                                   for r in rids]).float().cpu()
                for j, r in enumerate(rids):
                    rows[r].append(out[j])
            for r in rids:
                runner.free_request(r)
            for r in rids:
                s = distinct[src[r]]
                err = rel_err(torch.stack(rows[r]), w.plain_rows(src[r], range(len(s) - steps, len(s))))
                assert err < TOL["bfloat16"], (shape, r, n_req, err)
    finally:
        del w
        torch.cuda.empty_cache()


def test_the_engine_hands_back_the_weights_it_was_built_from(tmp_path):
    """``get_weight`` of a model drawn from a seed on the GPU gives the values that the same seed writes
    into a folder on the CPU, and a model loaded from that folder hands back what the file holds."""
    from helpers import TINY_B, make_folder, read_folder
    from reinfer_amd.engine import LLMEngine
    cfg = config_from_dict(TINY_B)
    eng = LLMEngine(config=cfg, seed=1, dtype="bfloat16", num_blocks=8)
    folder = make_folder(tmp_path, "B", "bfloat16")            # seed 1 as well
    _, stored = read_folder(folder)
    loaded = LLMEngine(folder, dtype="bfloat16", num_blocks=8)
    for name in ("model.embed_tokens.weight", "model.layers.2.self_attn.k_proj.weight",
                 "model.layers.0.post_attention_layernorm.weight", "lm_head.weight"):
        assert torch.equal(eng.get_weight(name).float(), stored[name]), name
        assert torch.equal(loaded.get_weight(name).float(), stored[name]), name
    with pytest.raises(KeyError):
        eng.get_weight("model.layers.9.mlp.up_proj.weight")
    # the GPU draws what the CPU draws, bit for bit, also across the pieces a large tensor is drawn in
    from reinfer_amd.weights import ParamDecl, random_tensor
    for decl in (ParamDecl("m.weight", (5000, 4099)), ParamDecl("v.weight", (4097,), init="norm", role="vector")):
        for dt in (torch.float32, torch.bfloat16):
            assert torch.equal(random_tensor(decl, 3, dt, torch.device("cuda:0")).cpu(), random_tensor(decl, 3, dt)), decl.name


@pytest.fixture(scope="module")
def w8_long():
    """One layer of the 8B widths with room for positions up to 8,700."""
    SHAPES["8b_long"] = dict(raw_config(1, 4096, 32, 12288, False), max_position_embeddings=8704)
    w = Width("8b_long", max_tokens=8704, max_seqs=4)
    yield w
    del w
    torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_of_thousands_of_tokens_at_the_8b_widths(w8_long, dtype):
    """Steps longer than any other test feeds, at the rows where the dispatch changes: 8,192 tokens in one
    step (what the bench's 8,192-token prompt point runs: the output and down projections no longer add into the
    stream through the library, four times the query tiles the chip holds at once, the row kernels at 8,192 rows)
    from position 0 and behind 300 cached tokens; 4,096; and 3,072 and 3,073 rows, the last step whose library
    products add into the stream and the first whose do not, each from position 0 and behind earlier context.
    Logits at the first and last row of every step and at a spread between, against the plain implementation."""
    n = 8492
    seqs = {"xl": w8_long.seq("xl", n, 41)}
    plans = [[8192, 300], [300, 8192], [3072, 3073, 2347], [3073, 4096, 1323]]
    edges = set()
    for plan in plans:
        at = 0
        for k in plan:
            edges |= {at, at + 1, at + k - 1}
            at += k
    wanted = {"xl": sorted(edges | {63, 64, 1000, 2047, 2048, 4095, 4500, 5555, 6143, 6144, 7000, 8000, 8191, n - 2})}
    for plan in plans:
        check(w8_long, dtype, seqs, [[("xl", k)] for k in plan], wanted)


def test_decoding_requests_beside_two_prompt_portions_at_the_8b_widths(w8):
    """The step a serving run makes all the time: ten (then eight) requests decode while two others bring
    portions of their prompts, several steps in a row; with eight or more single tokens beside prompt tiles the
    decode attention runs on a second stream beside the prompt attention. Two decoding requests end in the
    middle and a new prompt starts on their blocks (the allocator hands the last freed out first); the keys and
    values of every freed block are overwritten with NaN at once, so a read of a stale slot shows."""
    for dtype in ("bfloat16", "float32"):
        runner = w8.runners[dtype]
        runner.poison_freed_blocks(True)
        try:
            dec = {f"d{i}": w8.seq(f"d{i}", 200 + 13 * i + 12, 60 + i) for i in range(10)}
            pro = {"p1": w8.seq("p1", 700, 71), "p2": w8.seq("p2", 500, 72), "p3": w8.seq("p3", 450, 73)}
            seqs = dict(dec, **pro)
            tail = 12                                         # each decoding request's last 12 tokens come one by one
            plan = [[(r, len(s) - tail) for r, s in list(dec.items())[lo:lo + 5]] for lo in (0, 5)]
            ones = [(r, 1) for r in dec]
            plan += [ones + [("p1", 256), ("p2", 200)], ones + [("p1", 256), ("p2", 200)],
                     ones + [("p1", 187), ("p2", 99)], ones + [("p1", 1), ("p2", 1)]]
            # d0 and d1 are cut short here: they end (in `ends`) and p3 starts on their blocks
            ones8 = [(r, 1) for r in dec if r not in ("d0", "d1")]
            plan += [ones8 + [("p3", 300)], ones8 + [("p3", 148)]] + [ones8 + [("p3", 1)]] * 2
            plan += [ones8] * 4
            wanted = {r: list(range(len(s) - tail, len(s))) for r, s in dec.items()}
            wanted["d0"] = wanted["d0"][:4]
            wanted["d1"] = wanted["d1"][:4]
            wanted.update({"p1": [0, 255, 256, 511, 512, 698, 699], "p2": [0, 199, 200, 399, 400, 498, 499],
                           "p3": [0, 1, 299, 300, 447, 448, 449]})
            short = dict(seqs, d0=seqs["d0"][:len(seqs["d0"]) - tail + 4], d1=seqs["d1"][:len(seqs["d1"]) - tail + 4])
            got = feed(runner, short, plan, wanted)
            for r in seqs:
                err = rel_err(got[r], w8.plain_rows(r, wanted[r]))
                assert err < TOL[dtype], (r, dtype, err)
            runner.manager.check()
        finally:
            runner.poison_freed_blocks(False)


def test_a_16384_token_prompt_in_one_step_at_the_32b_widths():
    """The longest step the bench times: a 16,384-token prompt as one step through one layer of the Qwen3-32B
    widths (64 query heads in groups of 8, so two workgroups a query tile and KV head; 256 query tiles; the
    library's products and the row kernels at 16,384 rows), bfloat16, then a few tokens one by one behind
    it. Logits at a spread of rows against the plain implementation."""
    SHAPES["32b_long"] = dict(raw_config(1, 5120, 64, 25600, False), max_position_embeddings=16640)
    w = Width("32b_long", max_tokens=16640, max_seqs=2)
    try:
        n = 16384 + 6
        seqs = {"xxl": w.seq("xxl", n, 51)}
        wanted = {"xxl": sorted({0, 1, 63, 64, 127, 128, 1000, 4095, 4096, 8191, 8192, 12000, 16319, 16320, 16382, 16383}
                                | set(range(16384, n)))}
        check(w, "bfloat16", seqs, [[("xxl", 16384)]] + [[("xxl", 1)]] * 6, wanted)
    finally:
        del w
        torch.cuda.empty_cache()
