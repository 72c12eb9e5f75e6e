"""An architecture none of whose layers keeps keys, with a position encoding that is added to the
embeddings, defined here and run through the public entry point with its default limits: no block
pool is made, requests are admitted by state slots alone, and a prompt longer than any block count
that would stand in for "no pool" goes through. Nothing in the framework's files knows these parts."""
import pytest
import torch

from kernel_double import KernelDouble
from reinfer_amd import kernels
from reinfer_amd.config import config_from_dict, register_architecture
from reinfer_amd.config.schema import BlockSpec, FeedForwardSpec, MixerSpec, ModelSpec, NormSpec, PositionSpec, RunEntry
from reinfer_amd.engine import LLMEngine
from reinfer_amd.models import declare_params
from reinfer_amd.parts import register_position
from reinfer_amd.sampling import SamplingParams
from reinfer_amd.weights import ParamDecl, random_tensors
from test_toy_mixer import DecayedSum, DecayedSumParams  # noqa: F401  (registers the mixer "toy_decayed_sum")

import plain_qwen3 as plain


@register_position("toy_learned_absolute")
class LearnedAbsolute:
    """A row of a table per position, added to the token's embedding."""

    @classmethod
    def declare_input_params(cls, spec, prefix):
        return [ParamDecl(prefix + "position_embeddings.weight", (spec.option("max_positions"), spec.option("hidden")))]

    def __init__(self, spec, device, weights=None, prefix="", dtype=None):
        self.table = weights[prefix + "position_embeddings.weight"]

    def add_to_stream(self, resid, batch):
        resid += self.table[batch.positions.long()].float()


RAW = {"hidden_size": 40, "intermediate_size": 72, "vocab_size": 211, "max_position_embeddings": 300,
       "rms_norm_eps": 2e-6, "decay": 0.6, "num_hidden_layers": 2}


class StateOnlyConfig:
    def __init__(self, raw):
        self.raw = dict(raw)

    @classmethod
    def from_dict(cls, raw):
        return cls(raw)

    def to_dict(self):
        return dict(self.raw, architectures=["ToyStateOnlyForCausalLM"])

    def to_spec(self):
        r = self.raw
        h = r["hidden_size"]
        norm = NormSpec("rmsnorm", h, r["rms_norm_eps"])
        ffn = FeedForwardSpec("swiglu", h, r["intermediate_size"])
        toy = MixerSpec("toy_decayed_sum", hidden=h, params=DecayedSumParams(decay=float(r["decay"])))
        blocks = tuple(BlockSpec("prenorm", toy, ffn, norm, norm, f"model.layers.{i}.", mixer_prefix="toy.")
                       for i in range(r["num_hidden_layers"]))
        pos = PositionSpec("toy_learned_absolute", extra=(("max_positions", r["max_position_embeddings"]), ("hidden", h)))
        return ModelSpec("ToyStateOnlyForCausalLM", r["vocab_size"], h, r["max_position_embeddings"], blocks,
                         tuple(RunEntry(i) for i in range(len(blocks))), norm, tie_embeddings=False,
                         input_position=pos)


def plain_forward(w, toks):
    D = torch.float64
    w = {k: v.to(D) for k, v in w.items()}
    eps = RAW["rms_norm_eps"]
    x = w["model.embed_tokens.weight"][torch.tensor(toks)] + w["model.position_embeddings.weight"][:len(toks)]
    for i in range(RAW["num_hidden_layers"]):
        p = f"model.layers.{i}."
        xn = plain.rms_norm(x, w[p + "input_layernorm.weight"], eps)
        s = torch.zeros(RAW["hidden_size"], dtype=D)
        ys = []
        for t in range(len(toks)):
            s = RAW["decay"] * s + xn[t]
            ys.append(w[p + "toy.mix.weight"] @ s)
        x = x + torch.stack(ys)
        xn = plain.rms_norm(x, w[p + "post_attention_layernorm.weight"], eps)
        x = x + plain.swiglu(xn, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return plain.rms_norm(x, w["model.norm.weight"], eps) @ w["lm_head.weight"].T


def plain_greedy(w, prompt, n):
    toks, out = list(prompt), []
    for _ in range(n):
        t = plain.argmax_first(plain_forward(w, toks)[-1])
        out.append(t)
        toks.append(t)
    return out


def check(device):
    register_architecture("ToyStateOnlyForCausalLM", StateOnlyConfig)
    cfg = config_from_dict(dict(RAW, architectures=["ToyStateOnlyForCausalLM"]))
    weights = random_tensors(declare_params(cfg.to_spec()), 5, torch.float32, std=0.1)
    assert "model.position_embeddings.weight" in weights
    eng = LLMEngine(config=cfg, dtype="float32", device=device, weights=weights)        # every limit at its default
    assert eng.runner.groups == [] and eng.runner.manager.stats()["blocks_total"] == []
    g = torch.Generator().manual_seed(1)
    prompts = [torch.randint(0, RAW["vocab_size"], (n,), generator=g).tolist() for n in (100, 7, 33)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o.finish_reason == "length"
        assert o.token_ids == plain_greedy(weights, p, 6), len(p)
    # more requests than state slots: the rest wait for a slot, nobody waits for a block
    eng2 = LLMEngine(config=cfg, dtype="float32", device=device, weights=weights, max_num_seqs=2,
                     max_num_batched_tokens=16)
    outs2 = eng2.generate(prompts, SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True))
    assert [o.token_ids for o in outs2] == [o.token_ids for o in outs]
    assert eng2.cache_stats()["preemptions"] == 0
    eng2.runner.manager.check()
    # the context still bounds a request
    with pytest.raises(Exception, match="context"):
        eng.add_request([1] * 300, SamplingParams(max_tokens=1))


def test_state_only_architecture_cpu():
    with kernels.use(KernelDouble()):
        check("cpu")


@pytest.mark.gpu
def test_state_only_architecture_gpu():
    assert kernels.current().name == "hip-gfx950"
    check("cuda:0")
