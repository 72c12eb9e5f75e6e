"""The plain implementation, pinned by what fixes it beside the reference's text:
vectors the reference's own tests hold, special cases that reduce to a library
routine, and invariants, each chosen so that a plausible mistake fails it."""
import math

import pytest
import torch

import plain_qwen3 as plain
from helpers import TINY_A, TINY_B, make_folder, random_tokens, read_folder

D = torch.float64


def test_rms_norm_vectors():
    """crates/kernels/src/refs.rs:168-178: [3,4] with w=[1,2], eps 0 -> [3,8]/sqrt(12.5); zero row -> 0."""
    y = plain.rms_norm(torch.tensor([3.0, 4.0], dtype=D), torch.tensor([1.0, 2.0], dtype=D), 0.0)
    assert torch.allclose(y, torch.tensor([3.0, 8.0], dtype=D) / math.sqrt(12.5))
    z = plain.rms_norm(torch.zeros(4, dtype=D), torch.ones(4, dtype=D), 1e-6)
    assert torch.equal(z, torch.zeros(4, dtype=D))
    # eps sits inside the root: a norm with eps outside gives 1/(0 + 1e-3), not 1/sqrt(1e-3)
    x = torch.full((8,), 1e-9, dtype=D)
    assert abs(plain.rms_norm(x, torch.ones(8, dtype=D), 1e-6)[0].item() - 1e-9 / math.sqrt(1e-18 + 1e-6)) < 1e-15
    # against the library routine
    x = torch.randn(5, 33, dtype=D)
    w = torch.rand(33, dtype=D)
    assert torch.allclose(plain.rms_norm(x, w, 1e-5), torch.nn.functional.rms_norm(x, (33,), w, 1e-5))


def test_head_norm_is_per_head():
    u = torch.randn(3, 4, 16, dtype=D)
    y = plain.head_norm(u, torch.ones(16, dtype=D), 0.0)
    assert torch.allclose((y * y).mean(dim=-1), torch.ones(3, 4, dtype=D))     # every head has RMS 1
    # a norm over all heads together would not
    u2 = u.clone()
    u2[:, 0] *= 10
    y2 = plain.head_norm(u2, torch.ones(16, dtype=D), 0.0)
    assert torch.allclose(y2[:, 1:], y[:, 1:])


def test_rope_vectors_and_invariants():
    """crates/kernels/src/refs.rs:181-192: position 0 is the identity; pair norms are
    kept for half=3, pos=7, theta=5000."""
    x = torch.tensor([[[1.0, -2.0, 0.5, 3.0, 0.25, -1.5]]], dtype=D)
    assert torch.allclose(plain.rope_neox(x, torch.tensor([0]), 5000.0), x)
    y = plain.rope_neox(x, torch.tensor([7]), 5000.0)
    for j in range(3):
        assert abs((y[0, 0, j] ** 2 + y[0, 0, j + 3] ** 2) - (x[0, 0, j] ** 2 + x[0, 0, j + 3] ** 2)) < 1e-12
    # the pairing is (j, j + half), and the sign: a complex multiplication by e^{i phi}
    d, pos, theta = 8, 5, 100.0
    u = torch.randn(1, 1, d, dtype=D)
    z = torch.complex(u[..., :4], u[..., 4:]) * torch.polar(
        torch.ones(4, dtype=D), pos * theta ** (-2.0 * torch.arange(4, dtype=D) / d))
    got = plain.rope_neox(u, torch.tensor([pos]), theta)
    assert torch.allclose(got[..., :4], z.real) and torch.allclose(got[..., 4:], z.imag)
    # only distances count
    q, k = torch.randn(1, 1, 16, dtype=D), torch.randn(1, 1, 16, dtype=D)
    def dot(p, t):
        return (plain.rope_neox(q, torch.tensor([p]), 1e4) * plain.rope_neox(k, torch.tensor([t]), 1e4)).sum()
    assert abs(dot(9, 4) - dot(109, 104)) < 1e-10
    assert abs(dot(9, 4) - dot(4, 9)) > 1e-6      # but the sign of the distance does


def test_attention_reduces_to_library_and_masks():
    T, H, d = 9, 3, 8
    q, k, v = (torch.randn(T, H, d, dtype=D) for _ in range(3))
    ref = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None], is_causal=True)[0].transpose(0, 1)
    assert torch.allclose(plain.causal_attention(q, k, v, 1 / math.sqrt(d)), ref)
    # grouped: query head a reads KV head a // ratio (14/2, 12/2: crates/cuda/tests/gqa_diff.rs:1-16)
    for Hq, Hkv in ((14, 2), (12, 2), (4, 4), (8, 1)):
        q = torch.randn(T, Hq, d, dtype=D)
        k, v = torch.randn(T, Hkv, d, dtype=D), torch.randn(T, Hkv, d, dtype=D)
        r = Hq // Hkv
        ref = torch.nn.functional.scaled_dot_product_attention(
            q.transpose(0, 1)[None], k.repeat_interleave(r, 1).transpose(0, 1)[None],
            v.repeat_interleave(r, 1).transpose(0, 1)[None], is_causal=True)[0].transpose(0, 1)
        assert torch.allclose(plain.causal_attention(q, k, v, 1 / math.sqrt(d)), ref)
    # one key: the output is its value; later keys never leak into earlier rows
    out = plain.causal_attention(q, k, v, 0.3)
    assert torch.allclose(out[0, 0], v[0, 0])
    k2, v2 = k.clone(), v.clone()
    k2[5:], v2[5:] = 99.0, -99.0
    assert torch.allclose(plain.causal_attention(q, k2, v2, 0.3)[:5], out[:5])
    # a window of W keeps keys p-W+1..p
    w3 = plain.causal_attention(q, k, v, 0.3, window=3)
    k3, v3 = k.clone(), v.clone()
    k3[:4], v3[:4] = 50.0, 50.0                   # positions 0..3 are outside the window of row 6
    assert torch.allclose(plain.causal_attention(q, k3, v3, 0.3, window=3)[6:], w3[6:])
    assert torch.allclose(plain.causal_attention(q, k, v, 0.3, window=T), out)


def test_swiglu():
    x = torch.randn(4, 6, dtype=D)
    wg, wu, wd = torch.randn(10, 6, dtype=D), torch.randn(10, 6, dtype=D), torch.randn(6, 10, dtype=D)
    F = torch.nn.functional
    assert torch.allclose(plain.swiglu(x, wg, wu, wd), F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd))
    assert torch.equal(plain.swiglu(x, torch.zeros_like(wg), wu, wd), torch.zeros(4, 6, dtype=D))   # gate 0 -> 0


def test_whole_model_special_cases(tmp_path):
    raw, w = read_folder(make_folder(tmp_path, "B", "float32"))
    toks = random_tokens(12, raw["vocab_size"], 1)
    full = plain.forward(raw, w, toks)
    # with the output and down projections zero, logits = head(norm(embedding))
    w0 = {k: (torch.zeros_like(v) if ("o_proj" in k or "down_proj" in k) else v) for k, v in w.items()}
    x = w["model.embed_tokens.weight"][torch.tensor(toks)].double()
    want = plain.rms_norm(x, w["model.norm.weight"].double(), raw["rms_norm_eps"]) @ w["lm_head.weight"].double().T
    assert torch.allclose(plain.forward(raw, w0, toks), want)
    # causal: a prefix's logits do not depend on what follows
    assert torch.allclose(plain.forward(raw, w, toks[:7]), full[:7])
    # a shift of all positions changes nothing (only distances count)
    assert torch.allclose(plain.forward(raw, w, toks, start_pos=37), full, atol=1e-9)
    # tied = untied with the head set to the embedding
    rawA, wA = read_folder(make_folder(tmp_path, "A", "float32"))
    toksA = random_tokens(9, rawA["vocab_size"], 2)
    untied = dict(rawA, tie_word_embeddings=False)
    wA2 = dict(wA)
    wA2["lm_head.weight"] = wA["model.embed_tokens.weight"]
    assert torch.equal(plain.forward(rawA, wA, toksA), plain.forward(untied, wA2, toksA))


def one_layer(raw, w):
    """The same model cut down to its first layer."""
    raw1 = dict(raw, num_hidden_layers=1)
    if "layer_types" in raw1:
        raw1["layer_types"] = raw1["layer_types"][:1]
    return raw1, {k: v for k, v in w.items() if not k.startswith("model.layers.") or k.startswith("model.layers.0.")}


def test_one_layer_in_closed_form(tmp_path):
    """Where the arrangement of a block shows in a formula that does not go through plain.forward's loop
    (crates/cuda/src/engine.rs:4075-4314): pre-norm blocks that add into the stream."""
    for which in ("A", "C"):
        raw, w = read_folder(make_folder(tmp_path / which, which, "float32"))
        raw1, w1 = one_layer(raw, w)
        eps = raw["rms_norm_eps"]
        dd = {k: v.double() for k, v in w1.items()}
        L = "model.layers.0."
        head = dd.get("lm_head.weight", dd["model.embed_tokens.weight"])
        toks = random_tokens(10, raw["vocab_size"], 3)
        x = dd["model.embed_tokens.weight"][torch.tensor(toks)]
        # the attention's output projection zero: x + mlp(norm2(x)), the second norm taken of the stream itself
        # (a norm of the block's output instead, or a feed-forward without the residual, gives something else)
        w_no_attn = dict(w1)
        w_no_attn[L + "self_attn.o_proj.weight"] = torch.zeros_like(w1[L + "self_attn.o_proj.weight"])
        y = x + plain.swiglu(plain.rms_norm(x, dd[L + "post_attention_layernorm.weight"], eps),
                             dd[L + "mlp.gate_proj.weight"], dd[L + "mlp.up_proj.weight"], dd[L + "mlp.down_proj.weight"])
        want = plain.rms_norm(y, dd["model.norm.weight"], eps) @ head.T
        assert torch.allclose(plain.forward(raw1, w_no_attn, toks), want, rtol=1e-9, atol=1e-9)
        # one token, the down projection zero: the softmax over one key is 1, so query, key, their norms and the
        # rotation drop out and head h returns the value of KV head h // (heads / KV heads), in head order
        w_no_mlp = dict(w1)
        w_no_mlp[L + "mlp.down_proj.weight"] = torch.zeros_like(w1[L + "mlp.down_proj.weight"])
        H, KV, d = raw["num_attention_heads"], raw["num_key_value_heads"], raw["head_dim"]
        x0 = x[:1]
        v = (plain.rms_norm(x0, dd[L + "input_layernorm.weight"], eps) @ dd[L + "self_attn.v_proj.weight"].T).view(KV, d)
        heads = torch.stack([v[h // (H // KV)] for h in range(H)]).reshape(1, H * d)
        y0 = x0 + heads @ dd[L + "self_attn.o_proj.weight"].T
        want0 = plain.rms_norm(y0, dd["model.norm.weight"], eps) @ head.T
        got0 = plain.forward(raw1, w_no_mlp, toks[:1], start_pos=5)
        assert torch.allclose(got0, want0, rtol=1e-9, atol=1e-9)
        # the other pairing of heads and KV heads (h % KV heads) is a different result for these weights
        if KV > 1 and H // KV > 1:
            wrong = torch.stack([v[h % KV] for h in range(H)]).reshape(1, H * d)
            assert not torch.allclose(wrong, heads)


def test_splitmix_vectors_and_greedy_ties():
    """crates/scheduler/src/rng.rs:83-87."""
    assert plain.splitmix64(0) == 0xE220A8397B1DCDAF
    assert plain.splitmix64(1) == 0x910A2DEC89025CC1
    assert plain.unit_from_u64((1 << 64) - 1) < 1.0 and plain.unit_from_u64(0) == 0.0
    assert plain.argmax_first(torch.tensor([1.0, 5.0, 5.0, 2.0])) == 1      # first maximum


def test_logit_bias_is_added_first_and_validated():
    """Reference semantics (crates/cuda/tests/sampler_gpu.rs:369-372): a bias of -5 on the
    favourite flips the greedy token to the runner-up; non-finite logits stay."""
    import pytest
    from reinfer_amd.sampling import SamplingParams
    logits = torch.tensor([0.0, 2.0, 3.0, float("-inf")])
    out = plain.filter_logits(logits, 0.0, logit_bias=((2, -5.0), (3, 100.0)))
    assert int(out.argmax()) == 1 and out[3] == float("-inf") and out[2] == -2.0
    p = SamplingParams(logit_bias={7: 1.5, 2: -1.0})
    assert p.logit_bias == ((2, -1.0), (7, 1.5)) and p.filters
    with pytest.raises(ValueError, match="twice"):
        SamplingParams(logit_bias=((1, 0.5), (1, 0.25)))
    assert not SamplingParams().filters


def test_rope_frequency_schedule_by_hand():
    """The frequency of pair j is theta^(-2j/d) with d the whole head size (crates/kernels/src/refs.rs:25-37:
    ``exp = -(2 p) / (2 half)``; crates/cuda/tests/engine_vs_cpu.rs:291-299). The numbers below are written out,
    not computed from the same expression: theta^(-j/d), or d/2 in the denominator, gives others."""
    # d = 4, theta = 10000, position 1: frequencies [1, 0.01]
    e = torch.eye(4, dtype=D).view(4, 1, 4)
    y = plain.rope_neox(e, torch.tensor([1, 1, 1, 1]), 10000.0)[:, 0]
    cos1, sin1 = 0.5403023058681398, 0.8414709848078965
    cos001, sin001 = 0.9999500004166653, 0.009999833334166664
    want = torch.tensor([[cos1, 0.0, sin1, 0.0],          # unit vector 0: a = 1, b = 0 of pair 0
                         [0.0, cos001, 0.0, sin001],      # unit vector 1: pair 1 turns by 0.01, not by 1 or 0.1
                         [-sin1, 0.0, cos1, 0.0],         # unit vector 2 = b of pair 0: out[0] = -b sin
                         [0.0, -sin001, 0.0, cos001]], dtype=D)
    assert torch.allclose(y, want, rtol=0, atol=1e-15)
    # d = 8, theta = 10000, position 3, pair 3: frequency 10000^(-6/8) = 0.001, angle 0.003
    u = torch.zeros(1, 1, 8, dtype=D)
    u[0, 0, 3] = 1.0
    y = plain.rope_neox(u, torch.tensor([3]), 10000.0)[0, 0]
    assert abs(y[3].item() - 0.999995500003375) < 1e-15 and abs(y[7].item() - 0.002999995500002025) < 1e-15
    assert y[[0, 1, 2, 4, 5, 6]].abs().max().item() == 0.0
    # pair 1 of the same: 10000^(-2/8) = 0.1, angle 0.3
    u = torch.zeros(1, 1, 8, dtype=D)
    u[0, 0, 5] = 2.0
    y = plain.rope_neox(u, torch.tensor([3]), 10000.0)[0, 0]
    assert abs(y[1].item() + 2 * 0.29552020666133955) < 1e-15 and abs(y[5].item() - 2 * 0.955336489125606) < 1e-15


def _two_token_block(d_scale_q: float = 1.0):
    """One head of size 4, all projections the identity (q's scaled by ``d_scale_q``), norm weights 1."""
    eye = torch.eye(4, dtype=D)
    return {"L.self_attn.q_proj.weight": eye * d_scale_q, "L.self_attn.k_proj.weight": eye,
            "L.self_attn.v_proj.weight": eye, "L.self_attn.o_proj.weight": eye,
            "L.self_attn.q_norm.weight": torch.ones(4, dtype=D), "L.self_attn.k_norm.weight": torch.ones(4, dtype=D)}


def test_attention_scale_by_hand():
    """Two keys, weights softmax([a, b] / sqrt(d)) written out (crates/cuda/tests/engine_vs_cpu.rs:203,
    ``scale = 1 / sqrt(d)``, on the score before the softmax). Token 0 = [2,0,0,0] at position 0, token 1 =
    [0,0,2,0] at position 1 (theta 10000, d = 4: pair 0 turns by 1 radian). Head norm with eps 0 leaves both
    (mean square 1). q1 = k1 = [-2 sin 1, 0, 2 cos 1, 0], k0 = [2,0,0,0]: scores [-4 sin 1, 4], over sqrt(4):
    [-1.682941969615793, 2]; the weight of key 1 is 1 / (1 + exp(-3.682941969615793)) = 0.9754680718274085.
    Without the scale it would be 0.99937; with 1/d, 0.863."""
    xn = torch.tensor([[2.0, 0, 0, 0], [0, 0, 2.0, 0]], dtype=D)
    out = plain.attention_block(xn, torch.tensor([0, 1]), _two_token_block(), "L.", 1, 1, 4, 10000.0, 0.0, 0)
    p1 = 0.9754680718274085
    assert torch.allclose(out[0], xn[0], rtol=0, atol=1e-15)                 # one key: its value
    want = (1 - p1) * xn[0] + p1 * xn[1]                                     # values are not rotated
    assert torch.allclose(out[1], want, rtol=0, atol=1e-14), (out[1], want)


def test_head_norm_eps_is_the_layer_eps_by_hand():
    """The head norm's eps is rms_norm_eps, inside the root (crates/cuda/tests/engine_vs_cpu.rs:185-195 pass
    ``cfg.rms_eps``). Queries of order 1e-3 (q's projection scaled by 1e-3) make it count: q = [2e-3, 0, 0, 0]
    has mean square 1e-6, so with eps 1e-5 the normed q is 2e-3 / sqrt(1.1e-5) = 0.6030226891555273 (with
    eps 0, or 1e-6, it would be 2 or 1.414). Both tokens [2,0,0,0]; keys 2 / sqrt(1 + 1e-5) = 1.9999900000749994.
    Position 1 turns pair 0 by 1 radian: q1.k0 = |q||k| cos 1, q1.k1 = |q||k|; over sqrt(4) the scores differ
    by |q||k| (1 - cos 1) / 2 = 0.27720...; the weight of key 1 is 1 / (1 + exp(-that))."""
    w = _two_token_block(1e-3)
    # Both tokens are [2,0,0,0]; the values must still tell the keys apart: a 1e-30 in token 1's last entry
    # leaves norms and scores alone and is made 1 by the value projection. Values: token 0 [1,0,0,0], token 1 [1,1,0,0].
    xn2 = torch.tensor([[2.0, 0, 0, 0], [2.0, 0, 0, 1e-30]], dtype=D)
    vproj = torch.zeros(4, 4, dtype=D)
    vproj[0, 0] = 0.5
    vproj[1, 3] = 1e30
    w["L.self_attn.v_proj.weight"] = vproj
    out = plain.attention_block(xn2, torch.tensor([0, 1]), w, "L.", 1, 1, 4, 10000.0, 1e-5, 0)
    q_len, k_len = 0.6030226891555273, 1.9999900000749994
    gap = q_len * k_len * (1 - 0.5403023058681398) / 2.0
    p1 = 1.0 / (1.0 + math.exp(-gap))
    assert abs(out[1, 0].item() - 1.0) < 1e-12
    assert abs(out[1, 1].item() - p1) < 1e-9, (out[1, 1].item(), p1)
    assert abs(p1 - 0.5688) < 1e-3          # eps 0 would give 0.7149, eps 1e-6 0.6570
