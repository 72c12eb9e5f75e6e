"""A mixer with state of its own, defined here, is registered, built and stepped
without a change to the framework's files: the registries, the per-request state
slots and the run order are all it needs. The toy keeps a decayed sum of its
inputs per request; a model alternates it with attention, runs one block twice
and lets the second run read the first one's cache."""
from dataclasses import dataclass

import pytest
import torch

from kernel_double import KernelDouble
from reinfer_amd import kernels
from reinfer_amd.config import register_architecture
from reinfer_amd.config.schema import (BlockSpec, FeedForwardSpec, MixerSpec, ModelSpec, NormSpec, PositionSpec,
                                       RunEntry)
from reinfer_amd.engine import ModelRunner, StepEntry
from reinfer_amd.models import declare_params
from reinfer_amd.parts import StateNeed, register_mixer
from reinfer_amd.weights import ParamDecl, random_tensors

import plain_qwen3 as plain


@dataclass(frozen=True)
class DecayedSumParams:
    """The toy mixer's own typed record (MixerSpec.params): it has no heads and no head size."""
    decay: float


@register_mixer("toy_decayed_sum")
class DecayedSum:
    """s <- decay * s + x_t ;  y_t = s W^T. State: one vector per request."""

    @classmethod
    def declare_params(cls, spec, prefix):
        return [ParamDecl(prefix + "mix.weight", (spec.hidden, spec.hidden))]

    def __init__(self, spec, weights, prefix, dtype, device):
        self.w = weights[prefix + "mix.weight"]
        self.decay = spec.params.decay
        self.hidden = spec.hidden
        self.dtype = dtype

    def cache_need(self):
        return StateNeed((self.hidden,), torch.float32)

    def forward(self, x, batch, cache):
        out = torch.empty_like(x)
        slots = batch.state_slots.tolist()
        fresh = batch.fresh.tolist()
        t = 0
        for i, q in enumerate(batch.q_lens):
            s = torch.zeros(self.hidden, dtype=torch.float32, device=x.device) if fresh[i] \
                else cache.state[slots[i]].clone()
            for j in range(q):
                s = self.decay * s + x[t + j].float()
                out[t + j] = (self.w.float() @ s).to(self.dtype)
            cache.state[slots[i]] = s
            t += q
        return out


class ToyConfig:
    """hidden, heads and so on come from the dictionary, as for any architecture."""

    def __init__(self, raw):
        self.raw = dict(raw)

    @classmethod
    def from_dict(cls, raw):
        return cls(raw)

    def to_dict(self):
        return dict(self.raw, architectures=["ToyStateForCausalLM"])

    def to_spec(self):
        r = self.raw
        h, d = r["hidden_size"], r["head_dim"]
        norm = NormSpec("rmsnorm", h, r["rms_norm_eps"])
        ffn = FeedForwardSpec("swiglu", h, r["intermediate_size"])
        attn = MixerSpec("gqa_attention", hidden=h, num_heads=r["num_attention_heads"],
                         num_kv_heads=r["num_key_value_heads"], head_dim=d, scale=d ** -0.5, qk_norm=True,
                         qk_norm_eps=r["rms_norm_eps"], position=PositionSpec("rope_neox", d, r["rope_theta"]))
        toy = MixerSpec("toy_decayed_sum", hidden=h, params=DecayedSumParams(decay=float(r["decay"])))
        blocks = (BlockSpec("prenorm", attn, ffn, norm, norm, "model.layers.0."),
                  BlockSpec("prenorm", toy, ffn, norm, norm, "model.layers.1.", mixer_prefix="toy."),
                  BlockSpec("prenorm", attn, ffn, norm, norm, "model.layers.2."))
        # block 0 runs twice; its second run has a cache of its own; block 2 reads the first run's cache
        order = (RunEntry(0), RunEntry(1), RunEntry(0), RunEntry(2, cache_from=0))
        return ModelSpec("ToyStateForCausalLM", r["vocab_size"], h, r["max_position_embeddings"], blocks, order,
                         norm, tie_embeddings=True)


RAW = {"hidden_size": 48, "head_dim": 16, "num_attention_heads": 3, "num_key_value_heads": 1,
       "intermediate_size": 80, "vocab_size": 97, "max_position_embeddings": 128, "rms_norm_eps": 1e-6,
       "rope_theta": 10000.0, "decay": 0.7}


def plain_toy_forward(w, toks):
    """Whole sequence, no cache, from the formulas above and the plain parts."""
    D = torch.float64
    w = {k: v.to(D) for k, v in w.items()}
    eps, d, Hq, Hkv, theta = RAW["rms_norm_eps"], RAW["head_dim"], 3, 1, RAW["rope_theta"]
    pos = torch.arange(len(toks))
    x = w["model.embed_tokens.weight"][torch.tensor(toks)]

    def ffn(x, p):
        xn = plain.rms_norm(x, w[p + "post_attention_layernorm.weight"], eps)
        return x + plain.swiglu(xn, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])

    def qkv(x, p):
        xn = plain.rms_norm(x, w[p + "input_layernorm.weight"], eps)
        T = len(toks)
        q = plain.rope_neox(plain.head_norm((xn @ w[p + "self_attn.q_proj.weight"].T).reshape(T, Hq, d),
                                            w[p + "self_attn.q_norm.weight"], eps), pos, theta)
        k = plain.rope_neox(plain.head_norm((xn @ w[p + "self_attn.k_proj.weight"].T).reshape(T, Hkv, d),
                                            w[p + "self_attn.k_norm.weight"], eps), pos, theta)
        v = (xn @ w[p + "self_attn.v_proj.weight"].T).reshape(T, Hkv, d)
        return q, k, v

    def attn(x, p, kv=None):
        q, k, v = qkv(x, p)
        if kv is not None:
            k, v = kv
        o = plain.causal_attention(q, k, v, d ** -0.5).reshape(len(toks), Hq * d)
        return x + o @ w[p + "self_attn.o_proj.weight"].T, (k, v)

    x, kv0 = attn(x, "model.layers.0.")
    x = ffn(x, "model.layers.0.")
    xn = plain.rms_norm(x, w["model.layers.1.input_layernorm.weight"], eps)
    s = torch.zeros(RAW["hidden_size"], dtype=D)
    ys = []
    for t in range(len(toks)):
        s = RAW["decay"] * s + xn[t]
        ys.append(w["model.layers.1.toy.mix.weight"] @ s)
    x = ffn(x + torch.stack(ys), "model.layers.1.")
    x, _ = attn(x, "model.layers.0.")
    x = ffn(x, "model.layers.0.")
    x, _ = attn(x, "model.layers.2.", kv=kv0)
    x = ffn(x, "model.layers.2.")
    return plain.rms_norm(x, w["model.norm.weight"], eps) @ w["model.embed_tokens.weight"].T


def check(device):
    register_architecture("ToyStateForCausalLM", ToyConfig)
    from reinfer_amd.config import config_from_dict
    cfg = config_from_dict(dict(RAW, architectures=["ToyStateForCausalLM"]))
    spec = cfg.to_spec()
    weights = random_tensors(declare_params(spec), 3, torch.float32, std=0.08)
    runner = ModelRunner.from_config(cfg, dtype="float32", device=device, weights=weights, max_tokens=128,
                                     max_seqs=3)
    assert len(runner.groups) == 1 and runner.groups[0].entries == (0, 2)      # entry 3 reads entry 0
    assert runner.caches[1].state.shape == (3, 48) and runner.caches[3].k is runner.caches[0].k
    g = torch.Generator().manual_seed(0)
    seqs = {r: torch.randint(0, 97, (n,), generator=g).tolist() for r, n in (("a", 23), ("b", 31), ("c", 9), ("d", 12))}
    refs = {r: plain_toy_forward(weights, t).float() for r, t in seqs.items()}
    plan = [[("a", 5), ("b", 2)], [("a", 1), ("b", 20), ("c", 9)], [("a", 17), ("b", 1)],
            [("b", 8), ("d", 3)], [("d", 9)]]       # d reuses the state slot of a or c
    fed = {r: 0 for r in seqs}
    got = {r: [] for r in seqs}
    for items in plan:
        entries = []
        for r, n in items:
            if not runner.has_request(r):
                runner.add_request(r)
            entries.append(StepEntry(r, seqs[r][fed[r]:fed[r] + n], list(range(n))))
        out = runner.step(entries).float().cpu()
        o = 0
        for r, n in items:
            got[r].append(out[o:o + n])
            o += n
            fed[r] += n
            if fed[r] == len(seqs[r]):
                runner.free_request(r)
    for r in seqs:
        err = (torch.cat(got[r]) - refs[r]).abs().max() / refs[r].abs().max()
        assert err < 2e-5, (r, float(err))


def test_toy_mixer_bookkeeping_cpu():
    with kernels.use(KernelDouble()):
        check("cpu")


@pytest.mark.gpu
def test_toy_mixer_gpu():
    assert kernels.current().name == "hip-gfx950"
    check("cuda:0")
