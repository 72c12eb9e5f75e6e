"""Each part a layer is put together from, alone, against its plain formula, at sizes that
are not the tiny models': norm, position encoding with the mixer, feed-forward, block.
Then two toy parts defined here, a routed feed-forward and a position encoding of
its own, registered and run in a block without a change to the framework's files."""
import math

import pytest
import torch

import plain_qwen3 as plain
from reinfer_amd import kernels
from reinfer_amd.cache import CacheGroupSpec, CacheManager
from reinfer_amd.cache.layout import cache_shape
from reinfer_amd.config.schema import BlockSpec, FeedForwardSpec, MixerSpec, NormSpec, PositionSpec
from reinfer_amd.engine import StepEntry, build_step_batch
from reinfer_amd.parts import LayerCache, lookup, register_feed_forward, register_position
from reinfer_amd.weights import ParamDecl, random_tensors

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 2e-5, "bfloat16": 2e-2}


def rel(got, ref):
    got, ref = got.double().cpu(), ref.double().cpu()
    assert torch.isfinite(got).all()
    return float((got - ref).abs().max() / ref.abs().max())


def weights_for(decls, seed, dtype, std=0.05):
    """(tensors on the device in the compute dtype, the same values as float64 on the CPU)."""
    w = random_tensors(decls, seed, DT[dtype], std=std)
    return {k: v.to(DEV) for k, v in w.items()}, {k: v.double() for k, v in w.items()}


class OneRequest:
    """A cache manager, one layer's cache and the step batches of a single request."""

    def __init__(self, kv_heads, head_dim, dtype, tokens=256, block=16):
        self.manager = CacheManager([CacheGroupSpec(0, (0,))], block, [tokens // block], 2)
        shape = cache_shape(tokens // block, kv_heads, block, head_dim)
        self.cache = LayerCache(k=torch.full(shape, float("nan"), dtype=DT[dtype], device=DEV),
                                v=torch.full(shape, float("nan"), dtype=DT[dtype], device=DEV), group=0)
        self.manager.add("r")

    def batch(self, n):
        have = self.manager.get("r").num_tokens
        self.manager.grow("r", have + n)
        b = build_step_batch([StepEntry("r", [0] * n, [])], self.manager, DEV)
        self.manager.commit("r", have + n)
        return b


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_norm_part(dtype):
    spec = NormSpec("rmsnorm", 200, 3e-5)
    cls = lookup("norm", "rmsnorm")
    w, wd = weights_for(cls.declare_params(spec, "n.weight"), 1, dtype)
    part = cls(spec, w, "n.weight", DT[dtype], DEV)
    torch.manual_seed(0)
    resid = torch.randn(9, 200, device=DEV)
    delta = torch.randn(9, 200, device=DEV).to(DT[dtype])
    want = resid.double().cpu() + delta.double().cpu()
    rows = torch.tensor([8, 2], dtype=torch.int32, device=DEV)
    got_rows = part.add_norm(resid, delta, rows=rows)
    assert rel(got_rows, plain.rms_norm(want[[8, 2]], wd["n.weight"], 3e-5)) < TOL[dtype]
    got = part.add_norm(resid, delta)
    assert torch.allclose(resid.double().cpu(), want, atol=1e-6)          # the sum stays float
    assert rel(got, plain.rms_norm(want, wd["n.weight"], 3e-5)) < TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T", [3, 70])               # few rows: the fused product; many: product, then gate
def test_feed_forward_part(dtype, T):
    spec = FeedForwardSpec("swiglu", hidden=72, intermediate=136)
    cls = lookup("feed_forward", "swiglu")
    w, wd = weights_for(cls.declare_params(spec, "m."), 2, dtype, std=0.1)
    part = cls(spec, w, "m.", DT[dtype], DEV)
    torch.manual_seed(T)
    x = torch.randn(T, 72, device=DEV).to(DT[dtype])
    ref = plain.swiglu(x.double().cpu(), wd["m.gate_proj.weight"], wd["m.up_proj.weight"], wd["m.down_proj.weight"])
    assert rel(part.forward(x, None), ref) < TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("Hq,Hkv,d,window", [(6, 2, 32, 0), (5, 1, 48, 0), (4, 4, 64, 23)])
def test_attention_part_with_rotation(dtype, Hq, Hkv, d, window):
    """The mixer alone: a prompt in two portions, then single tokens, against the plain block
    on the whole sequence (rotation by absolute position, head norm before it, scale on the score)."""
    h, theta, eps = 88, 50000.0, 2e-6
    spec = MixerSpec("gqa_attention", hidden=h, num_heads=Hq, num_kv_heads=Hkv, head_dim=d, scale=d ** -0.5,
                     window=window, qk_norm=True, qk_norm_eps=eps, position=PositionSpec("rope_neox", d, theta))
    cls = lookup("mixer", "gqa_attention")
    w, wd = weights_for(cls.declare_params(spec, "self_attn."), 4, dtype, std=0.1)
    part = cls(spec, w, "self_attn.", DT[dtype], DEV)
    req = OneRequest(Hkv, d, dtype)
    torch.manual_seed(Hq)
    n = 90
    x = torch.randn(n, h, device=DEV).to(DT[dtype])
    ref = plain.attention_block(x.double().cpu(), torch.arange(n), wd, "", Hq, Hkv, d, theta, eps, window)
    outs, pos = [], 0
    for cut in (37, 45, 1, 1, 1, 5):
        outs.append(part.forward(x[pos:pos + cut].contiguous(), req.batch(cut), req.cache))
        pos += cut
    assert pos == n
    assert rel(torch.cat(outs), ref) < TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n", [40, 7, 100])     # up to 64 rows the projections add into the stream in their epilogues
def test_block_part(dtype, n):
    """Pre-norm arrangement: x += mixer(norm(x)); x += ffn(norm(x)), the last addend handed on."""
    h, Hq, Hkv, d, I, eps, theta = 80, 5, 1, 16, 104, 1e-5, 10000.0
    norm = NormSpec("rmsnorm", h, eps)
    spec = BlockSpec("prenorm",
                     MixerSpec("gqa_attention", hidden=h, num_heads=Hq, num_kv_heads=Hkv, head_dim=d, scale=d ** -0.5,
                               qk_norm=True, qk_norm_eps=eps, position=PositionSpec("rope_neox", d, theta)),
                     FeedForwardSpec("swiglu", h, I), norm, norm, "L.")
    cls = lookup("block", "prenorm")
    w, wd = weights_for(cls.declare_params(spec), 5, dtype, std=0.1)
    block = cls(spec, w, DT[dtype], DEV)
    req = OneRequest(Hkv, d, dtype)
    torch.manual_seed(1)
    x0 = torch.randn(n, h, device=DEV)
    resid = x0.clone()
    delta = block.forward(resid, None, req.batch(n), req.cache)     # None: the last part added in place
    got = resid.double().cpu() + (0 if delta is None else delta.double().cpu())
    x = x0.double().cpu()
    xn = plain.rms_norm(x, wd["L.input_layernorm.weight"], eps)
    x = x + plain.attention_block(xn, torch.arange(n), wd, "L.", Hq, Hkv, d, theta, eps, 0)
    xn = plain.rms_norm(x, wd["L.post_attention_layernorm.weight"], eps)
    x = x + plain.swiglu(xn, wd["L.mlp.gate_proj.weight"], wd["L.mlp.up_proj.weight"], wd["L.mlp.down_proj.weight"])
    assert rel(got, x) < TOL[dtype]


# ---------------------------------------------------------------- toy parts
@register_feed_forward("toy_top1_experts")
class Top1Experts:
    """Routing: each token goes to the expert with the largest router logit (float), scaled by
    that logit's sigmoid; an expert is a plain two-matrix ReLU network."""

    @classmethod
    def declare_params(cls, spec, prefix):
        E, h, I = dict(spec.extra)["experts"], spec.hidden, spec.intermediate
        out = [ParamDecl(prefix + "router.weight", (E, h))]
        for e in range(E):
            out += [ParamDecl(f"{prefix}experts.{e}.up.weight", (I, h)),
                    ParamDecl(f"{prefix}experts.{e}.down.weight", (h, I))]
        return out

    def __init__(self, spec, weights, prefix, dtype, device):
        self.E = dict(spec.extra)["experts"]
        self.router = weights[prefix + "router.weight"]
        self.up = [weights[f"{prefix}experts.{e}.up.weight"] for e in range(self.E)]
        self.down = [weights[f"{prefix}experts.{e}.down.weight"] for e in range(self.E)]
        self.dtype, self.spec = dtype, spec

    def forward(self, x, batch):
        ops = kernels.current()
        T = x.shape[0]
        logits = torch.empty((T, self.E), dtype=torch.float32, device=x.device)
        ops.linear(x, self.router, logits)                       # router logits in float
        choice = logits.argmax(dim=1)
        gate = torch.sigmoid(logits.gather(1, choice[:, None]))
        out = torch.zeros((T, self.spec.hidden), dtype=self.dtype, device=x.device)
        for e in range(self.E):
            idx = (choice == e).nonzero().flatten()
            if idx.numel() == 0:
                continue
            xe = x[idx].contiguous()
            mid = torch.empty((idx.numel(), self.spec.intermediate), dtype=self.dtype, device=x.device)
            ops.linear(xe, self.up[e], mid)
            mid = torch.relu(mid)
            ye = torch.empty((idx.numel(), self.spec.hidden), dtype=self.dtype, device=x.device)
            ops.linear(mid, self.down[e], ye)
            out[idx] = (ye.float() * gate[idx]).to(self.dtype)
        return out


@register_position("toy_rope_scaled")
class ScaledRotation:
    """Half-split rotation with every position divided by a factor: the mixer passes the
    constants to its kernel, so a scaled table of frequencies is all it takes."""
    style = 0

    def __init__(self, spec, device):
        self.rotary_dim = spec.rotary_dim
        j = torch.arange(spec.rotary_dim // 2, dtype=torch.float64)
        inv = torch.pow(torch.tensor(spec.theta, dtype=torch.float64), -2.0 * j / spec.rotary_dim) / 4.0
        self.inv_freq = inv.to(torch.float32).to(device)


def test_toy_routed_feed_forward_and_position_in_a_block():
    dtype = "float32"
    h, Hq, Hkv, d, I, E, eps, theta = 64, 4, 2, 16, 40, 3, 1e-6, 10000.0
    norm = NormSpec("rmsnorm", h, eps)
    spec = BlockSpec("prenorm",
                     MixerSpec("gqa_attention", hidden=h, num_heads=Hq, num_kv_heads=Hkv, head_dim=d, scale=d ** -0.5,
                               qk_norm=False, position=PositionSpec("toy_rope_scaled", d, theta)),
                     FeedForwardSpec("toy_top1_experts", h, I, extra=(("experts", E),)), norm, norm, "L.")
    cls = lookup("block", "prenorm")
    w, wd = weights_for(cls.declare_params(spec), 6, dtype, std=0.2)
    block = cls(spec, w, DT[dtype], DEV)
    req = OneRequest(Hkv, d, dtype)
    torch.manual_seed(2)
    n = 33
    x0 = torch.randn(n, h, device=DEV)
    # two portions: the rotation must follow absolute positions
    resid_a, resid_b = x0[:20].clone(), x0[20:].clone()
    da = block.forward(resid_a, None, req.batch(20), req.cache)
    db = block.forward(resid_b, None, req.batch(13), req.cache)
    assert da is not None and db is not None       # the toy feed-forward hands its addend back
    got = torch.cat([resid_a.double().cpu() + da.double().cpu(), resid_b.double().cpu() + db.double().cpu()])

    x = x0.double().cpu()
    xn = plain.rms_norm(x, wd["L.input_layernorm.weight"], eps)
    T = n
    q = (xn @ wd["L.self_attn.q_proj.weight"].T).reshape(T, Hq, d)
    k = (xn @ wd["L.self_attn.k_proj.weight"].T).reshape(T, Hkv, d)
    v = (xn @ wd["L.self_attn.v_proj.weight"].T).reshape(T, Hkv, d)
    # positions / 4 with the same base = rotation by a quarter of the angle
    half = d // 2
    j = torch.arange(half, dtype=torch.float64)
    ang = torch.arange(T, dtype=torch.float64)[:, None] * (theta ** (-2.0 * j / d) / 4.0)[None, :]

    def rot(u):
        a, b = u[..., :half], u[..., half:]
        c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
        return torch.cat([a * c - b * s, a * s + b * c], dim=-1)

    o = plain.causal_attention(rot(q), rot(k), v, d ** -0.5).reshape(T, Hq * d)
    x = x + o @ wd["L.self_attn.o_proj.weight"].T
    xn = plain.rms_norm(x, wd["L.post_attention_layernorm.weight"], eps)
    logits = xn @ wd["L.mlp.router.weight"].T
    choice = logits.argmax(dim=1)
    y = torch.zeros_like(x)
    for t in range(T):
        e = int(choice[t])
        mid = torch.relu(xn[t] @ wd[f"L.mlp.experts.{e}.up.weight"].T)
        y[t] = (mid @ wd[f"L.mlp.experts.{e}.down.weight"].T) * torch.sigmoid(logits[t, e])
    assert len(set(choice.tolist())) > 1           # the routing did route
    assert rel(got, x + y) < 5e-5
