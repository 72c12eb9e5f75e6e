"""Tiny configurations and helpers shared by the tests.

The configurations differ in every size and option: layers, width, query and KV
heads (2:1 groups, one KV head for eight, 2:1 with three groups), head size
(16, 32, 48; equal to width/heads or not), feed-forward width, vocabulary (no
power of two), rotation base, eps, tied or separate head, context, and a window
on some layers.
"""
from __future__ import annotations

import json
import os
from typing import Dict, List, Sequence

import torch

from reinfer_amd.config import config_from_dict
from reinfer_amd.weights import SafetensorsFile, write_model_folder

TINY_A = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
    "head_dim": 16, "intermediate_size": 192, "vocab_size": 512, "rope_theta": 10000.0,
    "rms_norm_eps": 1e-6, "tie_word_embeddings": True, "max_position_embeddings": 256,
    "attention_bias": False,
}
TINY_B = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 8, "num_key_value_heads": 1,
    "head_dim": 32, "intermediate_size": 320, "vocab_size": 1000, "rope_theta": 1000000.0,
    "rms_norm_eps": 1e-5, "tie_word_embeddings": False, "max_position_embeddings": 512,
    "attention_bias": False,
}
# a window on two of three layers, three KV groups, head size 48, odd vocabulary
TINY_C = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 3, "hidden_size": 80, "num_attention_heads": 6, "num_key_value_heads": 3,
    "head_dim": 48, "intermediate_size": 176, "vocab_size": 333, "rope_theta": 50000.0,
    "rms_norm_eps": 3e-6, "tie_word_embeddings": False, "max_position_embeddings": 384,
    "attention_bias": False, "sliding_window": 21, "use_sliding_window": True,
    "layer_types": ["sliding_attention", "full_attention", "sliding_attention"],
}
TINY = {"A": (TINY_A, 0), "B": (TINY_B, 1), "C": (TINY_C, 2)}


def make_folder(tmp_path, which: str, dtype: str = "bfloat16") -> str:
    raw, seed = TINY[which]
    cfg = config_from_dict(raw)
    out = os.path.join(str(tmp_path), f"tiny_{which}_{dtype}")
    if not os.path.isdir(out):
        write_model_folder(cfg, seed, out, dtype=dtype)
    return out


def read_folder(path: str):
    """(raw config dict, name -> float32 CPU tensor) for the plain implementation."""
    with open(os.path.join(path, "config.json")) as f:
        raw = json.load(f)
    with SafetensorsFile(os.path.join(path, "model.safetensors")) as sf:
        weights = {n: sf.tensor(n).float() for n in sf.names()}
    return raw, weights


def random_tokens(n: int, vocab: int, seed: int) -> List[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def rel_err(got: torch.Tensor, ref: torch.Tensor) -> float:
    """Largest difference over the largest reference magnitude (the row-max
    normalised drift of crates/cuda/tests/parity.rs:22-27)."""
    got, ref = got.double().cpu(), ref.double().cpu()
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert torch.isfinite(got).all(), "non-finite values"
    return float((got - ref).abs().max() / ref.abs().max().clamp_min(1e-30))


# Bounds, fixed by analysis and not by what passes:
#  float32: both sides sum in 32 or 64 bits in another order; a few hundred
#    roundings of 6e-8 each give ~1e-6 relative; 2e-5 leaves a margin of 10.
#  bfloat16: one rounding is 2^-9 = 2e-3 relative; about ten storage roundings a
#    layer, added in quadrature over at most 3 layers: 1.1e-2; 3e-2 is ~3 sigma.
TOL = {"float32": 2e-5, "bfloat16": 3e-2}
# The same metric for the bfloat16 engine against the float32 engine at the full depth of the Qwen3-8B shape
# (36 layers, the same bfloat16-rounded weights). By the argument above, ten roundings of 2^-9 a layer in
# quadrature over 36 layers are 3.7e-2 of the stream; a row's largest logit and the largest difference in that
# row are both about five standard deviations of their own distributions, so the metric's expected value is
# that figure itself. Measured once (a 2,048-token prompt, seven shorter ones, 32 decode steps of all eight):
# 0.045. Frozen at twice the expected figure; a fault that depth amplifies (a norm or a residual add in
# reduced precision, a product that rounds its partial sums) moves the drift by a factor, not by a fraction.
DEPTH_TOL = 0.075


def run_plan(runner, seqs: Dict[str, Sequence[int]], plan, ends=None, want_all: bool = True):
    """Feed ``seqs`` through ``runner`` as ``plan`` says and collect logits per request.

    ``plan`` is a list of steps, each a list of (request id, number of next tokens);
    ``ends`` maps a step index to the requests that finish after it (default: a
    request ends when all its tokens are fed). Returns {rid: logits [len, vocab]}.
    """
    from reinfer_amd.engine import StepEntry
    got = {r: [] for r in seqs}
    fed = {r: 0 for r in seqs}
    for step, items in enumerate(plan):
        entries = []
        for r, n in items:
            if not runner.has_request(r):
                runner.add_request(r)
            entries.append(StepEntry(r, list(seqs[r][fed[r]:fed[r] + n]), list(range(n))))
        out = runner.step(entries).float().cpu()
        o = 0
        for r, n in items:
            got[r].append(out[o:o + n])
            o += n
            fed[r] += n
        if ends is None:
            done = [r for r, _ in items if fed[r] == len(seqs[r])]
        else:
            done = ends.get(step, [])
        for r in done:
            runner.free_request(r)
        runner.manager.check()
    return {r: torch.cat(v) for r, v in got.items() if v}


def mixed_plan():
    """Six requests, four of them live in the third step, portions beside single tokens, 128 tokens of cache:
    the four that are live together fill all eight blocks of 16 between them, and the requests that come
    after them run on blocks that were given back."""
    lens = {"a": 30, "b": 20, "c": 30, "d": 20, "e": 40, "f": 25}
    plan = [
        [("a", 9), ("b", 2)],
        [("a", 1), ("b", 17), ("c", 5)],
        [("a", 20), ("b", 1), ("c", 12), ("d", 17)],
        [("c", 13), ("d", 3), ("e", 3)],
        [("e", 36), ("f", 2)],
        [("e", 1), ("f", 23)],
    ]
    return lens, plan
