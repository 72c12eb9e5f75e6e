"""One registry: architecture name -> configuration class.

A configuration class has ``from_dict(config_json) -> cfg``, ``cfg.to_dict()``
and ``cfg.to_spec() -> ModelSpec``. The name is ``architectures[0]`` of
config.json, else ``model_type`` (the reference selects the same way,
crates/arch/src/llama.rs:305-317).
"""
from __future__ import annotations

import json
import os
from typing import Any, Dict, Mapping, Tuple

from .schema import ConfigError, ModelSpec, UnknownArchitecture

_ARCHITECTURES: Dict[str, Any] = {}


def register_architecture(name: str, config_cls: Any, *aliases: str) -> None:
    for n in (name, *aliases):
        _ARCHITECTURES[n] = config_cls


def registered_architectures():
    return sorted(_ARCHITECTURES)


def architecture_name(cfg: Mapping[str, Any]) -> str:
    archs = cfg.get("architectures", None)
    if isinstance(archs, list) and archs and isinstance(archs[0], str):
        return archs[0]
    mt = cfg.get("model_type", None)
    if isinstance(mt, str):
        return mt
    raise ConfigError("architectures", "required key is missing")


def config_from_dict(cfg: Mapping[str, Any]):
    name = architecture_name(cfg)
    cls = _ARCHITECTURES.get(name)
    if cls is None:
        raise UnknownArchitecture(name, list(_ARCHITECTURES))
    return cls.from_dict(cfg)


def load_config(model_dir: str):
    """Read ``config.json`` (and ``generation_config.json`` for stop ids) of a folder."""
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise FileNotFoundError(f"{path}: a model folder holds config.json and model.safetensors")
    with open(path, "r", encoding="utf-8") as f:
        raw = json.load(f)
    if not isinstance(raw, dict):
        raise ConfigError("config.json", "expected a JSON object")
    gen_path = os.path.join(model_dir, "generation_config.json")
    if os.path.isfile(gen_path):
        # generation_config.json wins over config.json for stop ids
        # (crates/arch/src/llama.rs:406-432)
        with open(gen_path, "r", encoding="utf-8") as f:
            gen = json.load(f)
        if isinstance(gen, dict) and gen.get("eos_token_id") is not None:
            raw = dict(raw)
            raw["eos_token_id"] = gen["eos_token_id"]
    return config_from_dict(raw)
