"""Block arrangements, a paged cache tensor and a captured-step plan of the tests' own, registered here and
run through the public entry point without a change to the framework's files.

* ``toy_parallel``: one norm for both parts, x += mixer(n) + ffn(n); ``toy_mixer_only``: x += mixer(norm(x))
  and nothing else. Neither has the four parts of the "prenorm" arrangement; ``BlockSpec`` names only what
  they have, and each answers ``cache_need()`` itself.
* ``toy_latent_mean``: a mixer that keeps one small float vector a token in pages of its own shape
  (``PagedNeed``: an untiled ``[block_size, r]`` block), beside an attention layer's tiled keys and values in
  the same cache group, read through the same block tables.
* ``toy_prefix_mean``: a mixer whose work depends on a host-side number (how many positions to look at); for a
  captured decode step it fixes that number in ``plan_captured_step``.
Each architecture is compared with a plain whole-sequence form written from its formulas."""
from dataclasses import dataclass

import pytest
import torch

from kernel_double import KernelDouble
from reinfer_amd import kernels
from reinfer_amd.config import config_from_dict, register_architecture
from reinfer_amd.config.schema import (BlockSpec, FeedForwardSpec, MixerSpec, ModelSpec, NormSpec, PositionSpec,
                                       RunEntry)
from reinfer_amd.engine import LLMEngine, ModelRunner
from reinfer_amd.models import declare_params
from reinfer_amd.parts import PagedNeed, lookup, register_block, register_mixer
from reinfer_amd.sampling import SamplingParams
from reinfer_amd.weights import ParamDecl, random_tensors

import plain_qwen3 as plain
from helpers import run_plan


# --------------------------------------------------------------- arrangements
@register_block("toy_parallel")
class ParallelResidual:
    """x += mixer(n) + ffn(n), n = norm(x): one norm, both parts read it."""

    @classmethod
    def declare_params(cls, spec):
        p = spec.prefix
        return (lookup("norm", spec.mixer_norm.kind).declare_params(spec.mixer_norm, p + spec.mixer_norm_name)
                + lookup("mixer", spec.mixer.kind).declare_params(spec.mixer, p + spec.mixer_prefix)
                + lookup("feed_forward", spec.ffn.kind).declare_params(spec.ffn, p + spec.ffn_prefix))

    def __init__(self, spec, weights, dtype, device):
        p = spec.prefix
        assert spec.ffn_norm is None
        self.norm = lookup("norm", spec.mixer_norm.kind)(spec.mixer_norm, weights, p + spec.mixer_norm_name, dtype, device)
        self.token_mixer = lookup("mixer", spec.mixer.kind)(spec.mixer, weights, p + spec.mixer_prefix, dtype, device)
        self.feed_forward = lookup("feed_forward", spec.ffn.kind)(spec.ffn, weights, p + spec.ffn_prefix, dtype, device)
        self.graph_safe = bool(getattr(self.token_mixer, "graph_safe", False) and getattr(self.feed_forward, "graph_safe", False))
        self.scale = spec.params.ffn_scale

    def cache_need(self):
        return self.token_mixer.cache_need()

    def parts(self):
        return (self.norm, self.token_mixer, self.feed_forward)

    def forward(self, resid, delta, batch, cache):
        n = self.norm.add_norm(resid, delta)              # adds the block before's addend, then norms
        a = self.token_mixer.forward(n, batch, cache)
        f = self.feed_forward.forward(n, batch)
        return (a.float() + self.scale * f.float()).to(a.dtype)


@dataclass(frozen=True)
class ParallelParams:
    """The arrangement's own typed record (BlockSpec.params)."""
    ffn_scale: float


@register_block("toy_mixer_only")
class MixerOnly:
    """x += mixer(norm(x)); no feed-forward."""

    @classmethod
    def declare_params(cls, spec):
        p = spec.prefix
        return (lookup("norm", spec.mixer_norm.kind).declare_params(spec.mixer_norm, p + spec.mixer_norm_name)
                + lookup("mixer", spec.mixer.kind).declare_params(spec.mixer, p + spec.mixer_prefix))

    def __init__(self, spec, weights, dtype, device):
        p = spec.prefix
        self.norm = lookup("norm", spec.mixer_norm.kind)(spec.mixer_norm, weights, p + spec.mixer_norm_name, dtype, device)
        self.only = lookup("mixer", spec.mixer.kind)(spec.mixer, weights, p + spec.mixer_prefix, dtype, device)
        self.graph_safe = bool(getattr(self.only, "graph_safe", False))

    def cache_need(self):
        return self.only.cache_need() if hasattr(self.only, "cache_need") else None

    def parts(self):
        return (self.norm, self.only)

    def forward(self, resid, delta, batch, cache):
        return self.only.forward(self.norm.add_norm(resid, delta), batch, cache)


# --------------------------------------------------------------------- mixers
HOOK_CALLS = []


@register_mixer("toy_prefix_mean")
class PrefixMean:
    """y_t = W . mean of table[0 .. pos_t]: no cache, but its work is sized by a host-side number, the
    positions to look at. An eager step takes the step's longest context; a captured step must not, and
    is told the bucket's bound in ``plan_captured_step``."""
    graph_safe = True

    @classmethod
    def declare_params(cls, spec, prefix):
        return [ParamDecl(prefix + "table.weight", (spec.option("positions"), spec.hidden)),
                ParamDecl(prefix + "out.weight", (spec.hidden, spec.hidden))]

    def __init__(self, spec, weights, prefix, dtype, device):
        self.table = weights[prefix + "table.weight"]
        self.w = weights[prefix + "out.weight"]

    def plan_captured_step(self, batch, num_rows, ctx_cap):
        HOOK_CALLS.append((num_rows, ctx_cap))
        batch.extra["toy_prefix_cap"] = ctx_cap

    def forward(self, x, batch, cache):
        assert cache is None
        cap = min(batch.extra.get("toy_prefix_cap", batch.max_ctx_len), self.table.shape[0])
        pos = batch.positions.long()
        mask = (torch.arange(cap, device=x.device)[None, :] <= pos[:, None]).float()           # [T, cap]
        mean = (mask @ self.table[:cap].float()) / (pos + 1).float()[:, None]
        return ((mean + x.float()) @ self.w.float().T).to(x.dtype)


@register_mixer("toy_latent_mean")
class LatentMean:
    """Keeps c_t = W_in x_t (r floats a token) in pages; y_t = W_out . mean of c_0 .. c_t."""

    @classmethod
    def declare_params(cls, spec, prefix):
        r = spec.option("latent")
        return [ParamDecl(prefix + "in.weight", (r, spec.hidden)), ParamDecl(prefix + "out.weight", (spec.hidden, r))]

    def __init__(self, spec, weights, prefix, dtype, device):
        self.r = spec.option("latent")
        self.w_in, self.w_out = weights[prefix + "in.weight"], weights[prefix + "out.weight"]

    def cache_need(self):
        # one tensor, a block of it [block_size, r] float32 whatever the model's dtype
        return PagedNeed(tensors=(("latent", (-1, self.r), torch.float32),))

    def forward(self, x, batch, cache):
        pages = cache.tensors["latent"]                   # [blocks, block_size, r]
        assert cache.k is None and cache.v is None and pages.dtype == torch.float32
        bs = pages.shape[1]
        flat = pages.view(-1, self.r)
        lat = x.float() @ self.w_in.float().T
        slots = batch.slots[cache.group].long()
        keep = slots >= 0
        flat[slots[keep]] = lat[keep]
        table = batch.block_tables[cache.group].long()
        out = torch.empty_like(x)
        t = 0
        for i, (q, st) in enumerate(zip(batch.q_lens, batch.starts)):
            n = st + q
            idx = torch.arange(n, device=x.device)
            rows = flat[table[i, idx // bs] * bs + idx % bs]
            means = rows.cumsum(0)[st:n] / torch.arange(st + 1, n + 1, device=x.device)[:, None]
            out[t:t + q] = (means @ self.w_out.float().T).to(x.dtype)
            t += q
        return out


# ---------------------------------------------------------------- architectures
RAW = {"hidden_size": 48, "head_dim": 16, "num_attention_heads": 3, "num_key_value_heads": 1,
       "intermediate_size": 80, "vocab_size": 131, "max_position_embeddings": 160, "rms_norm_eps": 1e-6,
       "rope_theta": 10000.0, "ffn_scale": 0.5, "latent": 12}


def _attention(r):
    h, d = r["hidden_size"], r["head_dim"]
    return MixerSpec("gqa_attention", hidden=h, num_heads=r["num_attention_heads"],
                     num_kv_heads=r["num_key_value_heads"], head_dim=d, scale=d ** -0.5, qk_norm=True,
                     qk_norm_eps=r["rms_norm_eps"], position=PositionSpec("rope_neox", d, r["rope_theta"]))


class _Config:
    ARCH = ""

    def __init__(self, raw):
        self.raw = dict(raw)

    @classmethod
    def from_dict(cls, raw):
        return cls(raw)

    def to_dict(self):
        return dict(self.raw, architectures=[self.ARCH])


class ParallelConfig(_Config):
    ARCH = "ToyParallelForCausalLM"

    def to_spec(self):
        r = self.raw
        h = r["hidden_size"]
        norm = NormSpec("rmsnorm", h, r["rms_norm_eps"])
        ffn = FeedForwardSpec("swiglu", h, r["intermediate_size"])
        par = ParallelParams(ffn_scale=float(r["ffn_scale"]))
        prefix_mean = MixerSpec("toy_prefix_mean", hidden=h, extra=(("positions", r["max_position_embeddings"]),))
        blocks = (BlockSpec("toy_parallel", mixer=_attention(r), ffn=ffn, mixer_norm=norm, prefix="model.layers.0.", params=par),
                  BlockSpec("toy_mixer_only", mixer=prefix_mean, mixer_norm=norm, prefix="model.layers.1.", mixer_prefix="mean."),
                  BlockSpec("toy_parallel", mixer=_attention(r), ffn=ffn, mixer_norm=norm, prefix="model.layers.2.", params=par))
        return ModelSpec(self.ARCH, r["vocab_size"], h, r["max_position_embeddings"], blocks,
                         tuple(RunEntry(i) for i in range(3)), norm, tie_embeddings=True)


class LatentConfig(_Config):
    ARCH = "ToyLatentForCausalLM"

    def to_spec(self):
        r = self.raw
        h = r["hidden_size"]
        norm = NormSpec("rmsnorm", h, r["rms_norm_eps"])
        ffn = FeedForwardSpec("swiglu", h, r["intermediate_size"])
        latent = MixerSpec("toy_latent_mean", hidden=h, extra=(("latent", r["latent"]),))
        blocks = (BlockSpec("prenorm", latent, ffn, norm, norm, "model.layers.0.", mixer_prefix="lat."),
                  BlockSpec("prenorm", _attention(r), ffn, norm, norm, "model.layers.1."),
                  BlockSpec("toy_mixer_only", mixer=latent, mixer_norm=norm, prefix="model.layers.2.", mixer_prefix="lat."))
        return ModelSpec(self.ARCH, r["vocab_size"], h, r["max_position_embeddings"], blocks,
                         tuple(RunEntry(i) for i in range(3)), norm, tie_embeddings=True)


def _plain_attention(w, x, p, eps):
    r = RAW
    xn = plain.rms_norm(x, w[p + "input_layernorm.weight"], eps)
    a = plain.attention_block(xn, torch.arange(x.shape[0]), w, p, r["num_attention_heads"], r["num_key_value_heads"],
                              r["head_dim"], r["rope_theta"], eps, 0)
    return xn, a


def _plain_mlp(w, xn, p):
    return plain.swiglu(xn, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])


def plain_parallel(w, toks):
    w = {k: v.double() for k, v in w.items()}
    eps = RAW["rms_norm_eps"]
    x = w["model.embed_tokens.weight"][torch.tensor(toks)]
    T = len(toks)
    for p in ("model.layers.0.", "model.layers.2."):
        if p == "model.layers.2.":
            xn = plain.rms_norm(x, w["model.layers.1.input_layernorm.weight"], eps)
            table = w["model.layers.1.mean.table.weight"]
            means = table[:T].cumsum(0) / torch.arange(1, T + 1, dtype=torch.float64)[:, None]
            x = x + (means + xn) @ w["model.layers.1.mean.out.weight"].T
        xn, a = _plain_attention(w, x, p, eps)
        x = x + a + RAW["ffn_scale"] * _plain_mlp(w, xn, p)
    return plain.rms_norm(x, w["model.norm.weight"], eps) @ w["model.embed_tokens.weight"].T


def plain_latent(w, toks):
    w = {k: v.double() for k, v in w.items()}
    eps = RAW["rms_norm_eps"]
    x = w["model.embed_tokens.weight"][torch.tensor(toks)]
    T = len(toks)

    def latent(x, p):
        xn = plain.rms_norm(x, w[p + "input_layernorm.weight"], eps)
        c = xn @ w[p + "lat.in.weight"].T
        means = c.cumsum(0) / torch.arange(1, T + 1, dtype=torch.float64)[:, None]
        return means @ w[p + "lat.out.weight"].T

    def mlp(x, p):
        return _plain_mlp(w, plain.rms_norm(x, w[p + "post_attention_layernorm.weight"], eps), p)

    x = x + latent(x, "model.layers.0.")
    x = x + mlp(x, "model.layers.0.")
    x = x + _plain_attention(w, x, "model.layers.1.", eps)[1]
    x = x + mlp(x, "model.layers.1.")
    x = x + latent(x, "model.layers.2.")
    return plain.rms_norm(x, w["model.norm.weight"], eps) @ w["model.embed_tokens.weight"].T


def _greedy(forward, w, prompt, n):
    toks, out = list(prompt), []
    for _ in range(n):
        t = plain.argmax_first(forward(w, toks)[-1])
        out.append(t)
        toks.append(t)
    return out


# ---------------------------------------------------------------------- checks
def check_parallel(device):
    register_architecture(ParallelConfig.ARCH, ParallelConfig)
    cfg = config_from_dict(dict(RAW, architectures=[ParallelConfig.ARCH]))
    weights = random_tensors(declare_params(cfg.to_spec()), 4, torch.float32, std=0.1)
    assert "model.layers.0.post_attention_layernorm.weight" not in weights        # one norm a parallel block
    assert not any(k.startswith("model.layers.1.mlp") for k in weights)           # the middle layer only mixes
    g = torch.Generator().manual_seed(2)
    seqs = {r: torch.randint(0, RAW["vocab_size"], (n,), generator=g).tolist() for r, n in (("a", 37), ("b", 21), ("c", 50))}
    runner = ModelRunner.from_config(cfg, dtype="float32", device=device, weights=weights, max_tokens=96, max_seqs=3)
    # the middle entry keeps nothing: two of three entries share the one cache group
    assert [c is None for c in runner.caches] == [False, True, False] and runner.groups[0].entries == (0, 2)
    plan = [[("a", 20), ("b", 2)], [("a", 1), ("b", 19)], [("a", 16), ("c", 30)], [("c", 1)], [("c", 19)]]
    got = run_plan(runner, seqs, plan)
    for r, toks in seqs.items():
        ref = plain_parallel(weights, toks).float()
        err = (got[r] - ref).abs().max() / ref.abs().max()
        assert err < 2e-5, (r, float(err))
    # through the entry point, greedy, several requests decoding together
    eng = LLMEngine(config=cfg, dtype="float32", device=device, weights=weights, num_blocks=24, max_num_seqs=4)
    prompts = [seqs["a"][:9], seqs["b"][:17], seqs["c"][:5]]
    outs = eng.generate(prompts, SamplingParams(max_tokens=7, temperature=0.0, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o.token_ids == _greedy(plain_parallel, weights, p, 7), len(p)
    return eng


def check_latent(device):
    register_architecture(LatentConfig.ARCH, LatentConfig)
    cfg = config_from_dict(dict(RAW, architectures=[LatentConfig.ARCH]))
    weights = random_tensors(declare_params(cfg.to_spec()), 6, torch.float32, std=0.1)
    g = torch.Generator().manual_seed(3)
    seqs = {r: torch.randint(0, RAW["vocab_size"], (n,), generator=g).tolist()
            for r, n in (("a", 37), ("b", 21), ("c", 47), ("d", 33))}
    runner = ModelRunner.from_config(cfg, dtype="float32", device=device, weights=weights, max_tokens=96, max_seqs=3)
    # all three entries keep something a token and none has a window: one group, one block table a request
    assert len(runner.groups) == 1 and runner.groups[0].entries == (0, 1, 2)
    lat, att = runner.caches[0], runner.caches[1]
    assert set(lat.tensors) == {"latent"} and lat.tensors["latent"].shape == (6, 16, RAW["latent"])
    assert lat.k is None and set(att.tensors) == {"k", "v"} and att.k is att.tensors["k"]
    assert runner.caches[2].tensors["latent"] is not lat.tensors["latent"]
    runner.poison_freed_blocks(True)
    # 96 tokens of cache: c and d start on blocks that a and b gave back (and that read NaN since)
    plan = [[("a", 20), ("b", 2)], [("a", 1), ("b", 19)], [("a", 16), ("c", 30)], [("c", 1), ("d", 30)],
            [("c", 16), ("d", 3)]]
    got = run_plan(runner, seqs, plan)
    for r, toks in seqs.items():
        ref = plain_latent(weights, toks).float()
        err = (got[r] - ref).abs().max() / ref.abs().max()
        assert err < 2e-5, (r, float(err))
    eng = LLMEngine(config=cfg, dtype="float32", device=device, weights=weights, num_blocks=24, max_num_seqs=4)
    assert eng.runner.graphs is None            # the latent mixer does not say it can be captured
    prompts = [seqs["a"][:9], seqs["b"][:17]]
    outs = eng.generate(prompts, SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o.token_ids == _greedy(plain_latent, weights, p, 6), len(p)


def test_prenorm_block_names_what_it_misses():
    norm = NormSpec("rmsnorm", 48, 1e-6)
    spec = BlockSpec("prenorm", mixer=_attention(RAW), mixer_norm=norm, prefix="L.")
    with pytest.raises(ValueError, match="names no ffn, ffn_norm"):
        lookup("block", "prenorm")(spec, {}, torch.float32, torch.device("cpu"))


def test_block_arrangements_of_the_tests_own_cpu():
    with kernels.use(KernelDouble()):
        check_parallel("cpu")


def test_paged_tensor_of_a_mixers_own_shape_cpu():
    with kernels.use(KernelDouble()):
        check_latent("cpu")


@pytest.mark.gpu
def test_block_arrangements_of_the_tests_own_gpu():
    assert kernels.current().name == "hip-gfx950"
    del HOOK_CALLS[:]
    eng = check_parallel("cuda:0")
    # the decode steps of generate() were replayed from captured graphs, and the toy mixer was asked for its
    # plan once a bucket: three requests are padded to four rows, contexts to the model's limit of 160 (the
    # other bucket, one row, is the single-token step of the plan above)
    assert eng.runner.graphs is not None and eng.runner.graphs.replays >= 5
    assert sorted(HOOK_CALLS) == [(1, 160), (4, 160)], HOOK_CALLS


@pytest.mark.gpu
def test_paged_tensor_of_a_mixers_own_shape_gpu():
    assert kernels.current().name == "hip-gfx950"
    check_latent("cuda:0")
