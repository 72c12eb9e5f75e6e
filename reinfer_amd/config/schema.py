"""Typed descriptions of a model: what the parts are built from.

A configuration class (one per architecture) reads the architecture's own
``config.json`` keys and turns them into a :class:`ModelSpec`: a list of
blocks, each naming its mixer, feed-forward, norms and position encoding with
every size and constant as a field, plus the order in which the blocks run.
Parts are built from these records alone; none of them knows which model it
belongs to.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Mapping, Optional, Tuple


class ConfigError(ValueError):
    """A config.json key is missing or holds a value the engine cannot run.

    ``key`` names the offending key (the reference's ``ArchError::MissingKey``
    / ``InvalidValue`` carry the key the same way,
    crates/arch/src/llama.rs:122-173).
    """

    def __init__(self, key: str, why: str):
        super().__init__(f"config.json: {key}: {why}")
        self.key = key
        self.why = why


class UnknownArchitecture(ConfigError):
    def __init__(self, name: str, known: List[str]):
        ValueError.__init__(
            self, f"config.json: unknown architecture {name!r}; registered: {sorted(known)}")
        self.key = "architectures"
        self.why = "unknown architecture"
        self.name = name


# --------------------------------------------------------------------------
# key readers (fail closed, error names the key)
# --------------------------------------------------------------------------

_MISSING = object()


def read_int(cfg: Mapping[str, Any], key: str, default: Any = _MISSING, *, minimum: int = 0) -> int:
    v = cfg.get(key, None)
    if v is None:
        if default is _MISSING:
            raise ConfigError(key, "required key is missing")
        return default
    if isinstance(v, bool) or not isinstance(v, int):
        if isinstance(v, float) and float(v).is_integer():
            v = int(v)
        else:
            raise ConfigError(key, f"expected an integer, got {v!r}")
    if v < minimum:
        raise ConfigError(key, f"must be >= {minimum}, got {v}")
    return int(v)


def read_float(cfg: Mapping[str, Any], key: str, default: Any = _MISSING) -> float:
    v = cfg.get(key, None)
    if v is None:
        if default is _MISSING:
            raise ConfigError(key, "required key is missing")
        return default
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(key, f"expected a number, got {v!r}")
    v = float(v)
    if v != v or v in (float("inf"), float("-inf")):
        raise ConfigError(key, "must be finite")
    return v


def read_bool(cfg: Mapping[str, Any], key: str, default: bool) -> bool:
    v = cfg.get(key, None)
    if v is None:
        return default
    if not isinstance(v, bool):
        raise ConfigError(key, f"expected true/false, got {v!r}")
    return v


# --------------------------------------------------------------------------
# part specifications
# --------------------------------------------------------------------------

@dataclass(frozen=True)
class NormSpec:
    kind: str            # registry name of the norm part, e.g. "rmsnorm"
    size: int
    eps: float


@dataclass(frozen=True)
class PositionSpec:
    kind: str            # e.g. "rope_neox"; "none" for no position encoding
    rotary_dim: int = 0
    theta: float = 10000.0
    extra: Tuple[Tuple[str, Any], ...] = ()   # for position parts defined elsewhere

    def option(self, name: str, default: Any = None) -> Any:
        return dict(self.extra).get(name, default)


@dataclass(frozen=True)
class MixerSpec:
    """Token mixer of a block. ``kind`` picks the part; fields are its sizes."""
    kind: str                       # e.g. "gqa_attention"
    hidden: int
    num_heads: int = 0
    num_kv_heads: int = 0
    head_dim: int = 0
    scale: float = 0.0              # multiplies q.k before softmax
    window: int = 0                 # 0: all earlier keys; W>0: the last W keys
    qk_norm: bool = False           # per-head norm of q and k before rotation
    qk_norm_eps: float = 1e-6
    bias: bool = False
    position: PositionSpec = PositionSpec("none")
    extra: Tuple[Tuple[str, Any], ...] = ()   # for mixers defined elsewhere
    # A mixer that is not attention-shaped brings a record of its own (any frozen dataclass) with the
    # sizes and constants it needs, typed as it likes; the fields above then stay at their defaults.
    params: Any = None

    def option(self, name: str, default: Any = None) -> Any:
        return dict(self.extra).get(name, default)


@dataclass(frozen=True)
class FeedForwardSpec:
    kind: str                       # e.g. "swiglu"
    hidden: int
    intermediate: int
    extra: Tuple[Tuple[str, Any], ...] = ()
    params: Any = None              # a record of its own for a feed-forward defined elsewhere (experts, routing)


@dataclass(frozen=True)
class BlockSpec:
    """One layer: how norm, mixer and feed-forward are arranged, and its parts.

    The four part records are what the "prenorm" arrangement is built from; another arrangement may
    leave any of them out (one norm for both parts, a layer that only mixes) and bring a typed record
    of its own in ``params`` (any frozen dataclass), or loose options in ``extra``."""
    kind: str                       # e.g. "prenorm": x += mixer(norm(x)); x += ffn(norm(x))
    mixer: Optional[MixerSpec] = None
    ffn: Optional[FeedForwardSpec] = None
    mixer_norm: Optional[NormSpec] = None
    ffn_norm: Optional[NormSpec] = None
    prefix: str = ""                # tensor-name prefix of this block's weights
    mixer_prefix: str = "self_attn."
    ffn_prefix: str = "mlp."
    mixer_norm_name: str = "input_layernorm.weight"
    ffn_norm_name: str = "post_attention_layernorm.weight"
    params: Any = None
    extra: Tuple[Tuple[str, Any], ...] = ()

    def option(self, name: str, default: Any = None) -> Any:
        return dict(self.extra).get(name, default)


@dataclass(frozen=True)
class RunEntry:
    """One position in the run order.

    ``block`` indexes ``ModelSpec.blocks`` (a block may appear more than once:
    shared weights, separate cache). ``cache_from`` names an earlier run entry
    whose cache this entry reads instead of keeping one of its own.
    """
    block: int
    cache_from: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden: int
    max_positions: int
    blocks: Tuple[BlockSpec, ...]
    run_order: Tuple[RunEntry, ...]
    final_norm: NormSpec
    tie_embeddings: bool
    embed_name: str = "model.embed_tokens.weight"
    final_norm_name: str = "model.norm.weight"
    head_name: str = "lm_head.weight"
    eos_token_ids: Tuple[int, ...] = ()
    bos_token_id: Optional[int] = None
    # a position encoding that is added to the embeddings (learned or computed absolute positions), for
    # architectures whose mixers do not rotate; None: positions enter in the mixers only
    input_position: Optional[PositionSpec] = None
    input_position_prefix: str = "model."

    def __post_init__(self):
        for i, e in enumerate(self.run_order):
            if not 0 <= e.block < len(self.blocks):
                raise ConfigError("run_order", f"entry {i} names block {e.block} of {len(self.blocks)}")
            if e.cache_from is not None:
                if not 0 <= e.cache_from < i:
                    raise ConfigError("run_order", f"entry {i} reads the cache of entry {e.cache_from}, "
                                                   "which must come earlier")
                if self.run_order[e.cache_from].cache_from is not None:
                    raise ConfigError("run_order", f"entry {i} reads entry {e.cache_from}, "
                                                   "which has no cache of its own")
