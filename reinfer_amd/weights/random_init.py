"""Random-weights mode: a model folder from a configuration and a seed.

Every tensor has a generator of its own, seeded from (seed, tensor name), so a
tensor's values do not depend on which other tensors exist. Matrices and the
embedding are N(0, 0.02); norm weights U(0.8, 1.2). The reference has no such
mode (its tests need a real checkpoint, scripts/ci/ignored-tests.txt).
"""
from __future__ import annotations

import json
import os
from typing import Dict, Sequence

import torch

from .loader import INT_TABLE, MATRIX, VECTOR, ParamDecl
from .safetensors_io import write_safetensors

_MASK = (1 << 64) - 1


def splitmix64(x: int) -> int:
    """SplitMix64 one-shot mix (crates/scheduler/src/rng.rs:12-32)."""
    z = (x + 0x9E3779B97F4A7C15) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def _fnv1a(name: str) -> int:
    h = 0xCBF29CE484222325
    for b in name.encode("utf-8"):
        h = ((h ^ b) * 0x100000001B3) & _MASK
    return h


def tensor_seed(seed: int, name: str) -> int:
    return splitmix64((seed & _MASK) ^ _fnv1a(name)) & ((1 << 63) - 1)


def random_tensors(decls: Sequence[ParamDecl], seed: int, dtype: torch.dtype,
                   device: torch.device = torch.device("cpu"), std: float = 0.02) -> Dict[str, torch.Tensor]:
    """Values are drawn in float32 and rounded once to ``dtype``.

    The stream of a generator differs between device kinds, so a folder (always
    drawn on the CPU) is what makes a model reproducible, not the seed alone.
    """
    out: Dict[str, torch.Tensor] = {}
    for d in decls:
        if d.optional:
            continue
        g = torch.Generator(device=device)
        g.manual_seed(tensor_seed(seed, d.name))
        if d.init == "normal":
            t = torch.empty(d.shape, dtype=torch.float32, device=device).normal_(0.0, std, generator=g)
        elif d.init == "norm":
            t = torch.empty(d.shape, dtype=torch.float32, device=device).uniform_(0.8, 1.2, generator=g)
        elif d.init == "zeros":
            t = torch.zeros(d.shape, dtype=torch.float32, device=device)
        elif d.init == "int":
            t = torch.zeros(d.shape, dtype=torch.int32, device=device)
        else:
            raise ValueError(f"{d.name}: unknown init {d.init!r}")
        out[d.name] = t if d.role == INT_TABLE else t.to(dtype)
    return out


def write_model_folder(config, seed: int, out_dir: str, dtype: str = "bfloat16") -> str:
    """config.json + model.safetensors for ``config`` (any registered configuration)."""
    from ..models import declare_params   # parts own the list of tensors

    tdtype = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}[dtype]
    os.makedirs(out_dir, exist_ok=True)
    spec = config.to_spec()
    decls = declare_params(spec)
    tensors = random_tensors(decls, seed, tdtype)
    cfg = config.to_dict()
    cfg["torch_dtype"] = dtype
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg, f, indent=2)
    write_safetensors(os.path.join(out_dir, "model.safetensors"), tensors,
                      metadata={"format": "pt", "seed": str(seed)})
    return out_dir
