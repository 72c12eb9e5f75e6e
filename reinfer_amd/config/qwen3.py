"""Qwen3 dense decoder: typed configuration from its config.json keys.

Keys, defaults and error cases follow the reference's ``from_hf_config``
(crates/arch/src/llama.rs:304-396); ``tie_word_embeddings`` and the window keys
are read in addition (the reference never parses them,
crates/arch/src/llama.rs:304-396 has no such key).
"""
from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass, field
from typing import Any, Dict, List, Mapping, Optional, Tuple

from .schema import (BlockSpec, ConfigError, FeedForwardSpec, MixerSpec, ModelSpec, NormSpec,
                     PositionSpec, RunEntry, read_bool, read_float, read_int)

ARCHITECTURE = "Qwen3ForCausalLM"
MODEL_TYPE = "qwen3"


@dataclass(frozen=True)
class Qwen3Config:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    max_position_embeddings: int
    rope_theta: float
    rms_norm_eps: float
    tie_word_embeddings: bool
    # per layer: 0 = all earlier keys, W > 0 = the last W keys
    layer_windows: Tuple[int, ...]
    eos_token_ids: Tuple[int, ...] = ()
    bos_token_id: Optional[int] = None
    torch_dtype: str = "bfloat16"

    architecture: str = ARCHITECTURE

    # ---------------------------------------------------------------- reading
    @classmethod
    def from_dict(cls, cfg: Mapping[str, Any]) -> "Qwen3Config":
        # required sizes (llama.rs:319-337)
        max_pos = read_int(cfg, "max_position_embeddings", minimum=1)
        n_layer = read_int(cfg, "num_hidden_layers", minimum=1)
        hidden = read_int(cfg, "hidden_size", minimum=1)
        inter = read_int(cfg, "intermediate_size", minimum=1)
        vocab = read_int(cfg, "vocab_size", minimum=1)
        q_heads = read_int(cfg, "num_attention_heads", minimum=1)
        # optional with defaults (llama.rs:338-372)
        kv_heads = read_int(cfg, "num_key_value_heads", q_heads, minimum=0)
        if kv_heads == 0 or kv_heads > q_heads:
            raise ConfigError("num_key_value_heads", "kv heads must be in 1..=query heads")
        if q_heads % kv_heads != 0:
            raise ConfigError("num_key_value_heads",
                              f"{q_heads} query heads do not divide into {kv_heads} groups")
        head_dim = cfg.get("head_dim", None)
        if head_dim is None:
            if hidden % q_heads != 0:
                raise ConfigError("head_dim", "cannot derive head_dim from hidden_size/head_count")
            head_dim = hidden // q_heads
        else:
            head_dim = read_int(cfg, "head_dim", minimum=1)
        if head_dim % 2 != 0:
            raise ConfigError("head_dim", "rotation pairs (j, j + head_dim/2) need an even head_dim")
        theta = read_float(cfg, "rope_theta", 1_000_000.0)   # Qwen default, llama.rs:50-55
        if theta <= 0.0:
            raise ConfigError("rope_theta", "rope theta must be finite and > 0")
        eps = read_float(cfg, "rms_norm_eps", 1e-5)          # llama.rs:371-372
        if eps < 0.0:
            raise ConfigError("rms_norm_eps", "must be >= 0")
        tie = read_bool(cfg, "tie_word_embeddings", False)

        # what the engine has no part for must be off, not silently ignored
        if read_bool(cfg, "attention_bias", False):
            raise ConfigError("attention_bias", "Qwen3 projections carry no bias; true is not supported")
        act = cfg.get("hidden_act", None)
        if act is not None and act != "silu":
            # the gate of the feed-forward is SiLU in every kernel (the reference fixes it the same way,
            # crates/cuda/kernels/dense_kernels.cu:202-213, and never reads the key)
            raise ConfigError("hidden_act", f"the feed-forward's gate is SiLU; {act!r} is not supported")
        scaling = cfg.get("rope_scaling", None)
        if scaling not in (None, {}):
            kind = scaling.get("rope_type", scaling.get("type")) if isinstance(scaling, dict) else scaling
            if kind not in (None, "default"):
                raise ConfigError("rope_scaling", f"scaled rotation {kind!r} is not supported")

        windows = cls._read_windows(cfg, n_layer)

        eos = cls._read_ids(cfg, "eos_token_id")
        bos = cfg.get("bos_token_id", None)
        bos = int(bos) if isinstance(bos, int) and not isinstance(bos, bool) else None
        dtype = cfg.get("torch_dtype", cfg.get("dtype", "bfloat16"))
        if not isinstance(dtype, str):
            raise ConfigError("torch_dtype", f"expected a string, got {dtype!r}")
        return cls(vocab_size=vocab, hidden_size=hidden, intermediate_size=inter,
                   num_hidden_layers=n_layer, num_attention_heads=q_heads,
                   num_key_value_heads=kv_heads, head_dim=head_dim,
                   max_position_embeddings=max_pos, rope_theta=theta, rms_norm_eps=eps,
                   tie_word_embeddings=tie, layer_windows=windows, eos_token_ids=eos,
                   bos_token_id=bos, torch_dtype=dtype)

    @staticmethod
    def _read_ids(cfg: Mapping[str, Any], key: str) -> Tuple[int, ...]:
        """Scalar or list, every entry stops (the reference takes the first of a
        list only, llama.rs:411-418)."""
        v = cfg.get(key, None)
        if v is None:
            return ()
        if isinstance(v, int) and not isinstance(v, bool):
            return (int(v),)
        if isinstance(v, list) and all(isinstance(x, int) and not isinstance(x, bool) for x in v):
            return tuple(int(x) for x in v)
        raise ConfigError(key, f"expected an id or a list of ids, got {v!r}")

    @staticmethod
    def _read_windows(cfg: Mapping[str, Any], n_layer: int) -> Tuple[int, ...]:
        """Window of each layer from ``layer_types`` / ``sliding_window`` /
        ``use_sliding_window`` / ``max_window_layers``.

        ``layer_types`` (one of "full_attention" / "sliding_attention" per
        layer) wins; otherwise ``use_sliding_window`` turns the window on for
        layers with index >= ``max_window_layers``.
        """
        use = read_bool(cfg, "use_sliding_window", False)
        types = cfg.get("layer_types", None)
        window = cfg.get("sliding_window", None)
        if window is not None:
            window = read_int(cfg, "sliding_window", minimum=1)
        if types is not None:
            if not isinstance(types, list) or len(types) != n_layer:
                raise ConfigError("layer_types", f"expected a list of {n_layer} layer kinds")
            out = []
            for i, t in enumerate(types):
                if t == "full_attention":
                    out.append(0)
                elif t == "sliding_attention":
                    if window is None:
                        raise ConfigError("sliding_window", f"layer {i} is sliding_attention but no window is given")
                    out.append(window)
                else:
                    raise ConfigError("layer_types", f"layer {i}: unknown kind {t!r}")
            return tuple(out)
        if not use:
            return tuple(0 for _ in range(n_layer))
        if window is None:
            raise ConfigError("sliding_window", "use_sliding_window is true but no window is given")
        first = read_int(cfg, "max_window_layers", n_layer, minimum=0)
        return tuple(window if i >= first else 0 for i in range(n_layer))

    # ---------------------------------------------------------------- writing
    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architectures": [ARCHITECTURE],
            "model_type": MODEL_TYPE,
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "max_position_embeddings": self.max_position_embeddings,
            "rope_theta": self.rope_theta,
            "rms_norm_eps": self.rms_norm_eps,
            "tie_word_embeddings": self.tie_word_embeddings,
            "attention_bias": False,
            "hidden_act": "silu",
            "torch_dtype": self.torch_dtype,
        }
        if any(self.layer_windows):
            w = max(self.layer_windows)
            d["sliding_window"] = w
            d["use_sliding_window"] = True
            d["layer_types"] = ["sliding_attention" if x else "full_attention" for x in self.layer_windows]
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids) if len(self.eos_token_ids) > 1 else self.eos_token_ids[0]
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        return d

    # ---------------------------------------------------------------- the model
    def to_spec(self) -> ModelSpec:
        """Blocks and run order of the Qwen3 dense decoder.

        Pre-norm residual blocks; GQA attention with per-head q/k RMSNorm
        before NEOX rotation over the full head_dim, scale 1/sqrt(head_dim);
        SwiGLU feed-forward (crates/cuda/src/engine.rs:3970-4356).
        """
        blocks: List[BlockSpec] = []
        for i in range(self.num_hidden_layers):
            mixer = MixerSpec(
                kind="gqa_attention", hidden=self.hidden_size,
                num_heads=self.num_attention_heads, num_kv_heads=self.num_key_value_heads,
                head_dim=self.head_dim, scale=1.0 / math.sqrt(self.head_dim),
                window=self.layer_windows[i], qk_norm=True, qk_norm_eps=self.rms_norm_eps,
                bias=False,
                position=PositionSpec("rope_neox", rotary_dim=self.head_dim, theta=self.rope_theta))
            ffn = FeedForwardSpec(kind="swiglu", hidden=self.hidden_size,
                                  intermediate=self.intermediate_size)
            norm = NormSpec("rmsnorm", self.hidden_size, self.rms_norm_eps)
            blocks.append(BlockSpec(kind="prenorm", mixer=mixer, ffn=ffn, mixer_norm=norm,
                                    ffn_norm=norm, prefix=f"model.layers.{i}."))
        return ModelSpec(
            architecture=ARCHITECTURE, vocab_size=self.vocab_size, hidden=self.hidden_size,
            max_positions=self.max_position_embeddings, blocks=tuple(blocks),
            run_order=tuple(RunEntry(i) for i in range(self.num_hidden_layers)),
            final_norm=NormSpec("rmsnorm", self.hidden_size, self.rms_norm_eps),
            tie_embeddings=self.tie_word_embeddings,
            eos_token_ids=self.eos_token_ids, bos_token_id=self.bos_token_id)
