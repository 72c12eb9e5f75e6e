"""Random-weights mode: a model folder from a configuration and a seed.

Every element is a function of (seed, tensor name, index): a tensor's values do
not depend on which other tensors exist or on the device that draws them.
Matrices and the embedding are bell-shaped with deviation 0.02; norm weights
uniform on [0.8, 1.2). The reference has no such
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


_CHUNK = 1 << 24        # elements drawn at a time: bounds the temporaries of a large matrix


def _mix(z: torch.Tensor) -> torch.Tensor:
    """The finalising stage of SplitMix64 on int64 tensors (products wrap, shifts made logical by a mask)."""
    z = (z ^ ((z >> 30) & 0x3FFFFFFFF)) * -0x40A7B892E31B1A47         # 0xBF58476D1CE4E5B9 as a signed value
    z = (z ^ ((z >> 27) & 0x1FFFFFFFFF)) * -0x6B2FB644ECCEEE15         # 0x94D049BB133111EB
    return z ^ ((z >> 31) & 0x1FFFFFFFF)


def _signed(x: int) -> int:
    x &= _MASK
    return x - (1 << 64) if x >= (1 << 63) else x


def _draw(n: int, seed: int, kind: str, device: torch.device, std: float) -> torch.Tensor:
    """Element i of a tensor is a function of (seed, i) alone, made of integer operations and one float
    product, so the CPU and the GPU draw the same bits. "normal": the sum of eight 16-bit fields of two
    hashed words, centred and scaled to the standard deviation (a bell over +-4.9 deviations);
    "uniform": 24 bits over [0.8, 1.2)."""
    out = torch.empty(n, dtype=torch.float32, device=device)
    for lo in range(0, n, _CHUNK):
        hi = min(n, lo + _CHUNK)
        i = torch.arange(lo, hi, dtype=torch.int64, device=device)
        a = _mix(i * 2 + _signed(seed) + _signed(0x9E3779B97F4A7C15))
        if kind == "normal":
            b = _mix(i * 2 + 1 + _signed(seed) + _signed(0x9E3779B97F4A7C15))
            s = torch.zeros_like(i)
            for word in (a, b):
                for shift in (0, 16, 32, 48):
                    s += (word >> shift) & 0xFFFF
            # eight uniform fields on 0..65535: mean 4 * 65535, variance 8 * (65536^2 - 1) / 12
            scale = std / (((65536.0 ** 2 - 1.0) * 8.0 / 12.0) ** 0.5)
            out[lo:hi] = (s - 4 * 65535).to(torch.float32) * scale
        else:
            out[lo:hi] = 0.8 + ((a >> 40) & 0xFFFFFF).to(torch.float32) * (0.4 / 16777216.0)
    return out


def random_tensor(decl: ParamDecl, seed: int, dtype: torch.dtype,
                  device: torch.device = torch.device("cpu"), std: float = 0.02) -> torch.Tensor:
    """One declared tensor of the random model of ``seed``: drawn in float32, rounded once to ``dtype``;
    the same values on every device."""
    n = 1
    for v in decl.shape:
        n *= int(v)
    if decl.init == "normal":
        t = _draw(n, tensor_seed(seed, decl.name), "normal", device, std).view(decl.shape)
    elif decl.init == "norm":
        t = _draw(n, tensor_seed(seed, decl.name), "uniform", device, std).view(decl.shape)
    elif decl.init == "zeros":
        t = torch.zeros(decl.shape, dtype=torch.float32, device=device)
    elif decl.init == "int":
        t = torch.zeros(decl.shape, dtype=torch.int32, device=device)
    else:
        raise ValueError(f"{decl.name}: unknown init {decl.init!r}")
    return t if decl.role == INT_TABLE else t.to(dtype)


def random_tensors(decls: Sequence[ParamDecl], seed: int, dtype: torch.dtype,
                   device: torch.device = torch.device("cpu"), std: float = 0.02) -> Dict[str, torch.Tensor]:
    """Every declared tensor (but the optional ones) of the random model of ``seed``. A value depends on
    the seed, the tensor's name and the element's index, not on the device or on what else is drawn: a
    model drawn on the GPU is the one a folder written on the CPU holds."""
    return {d.name: random_tensor(d, seed, dtype, device, std) for d in decls if not d.optional}


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
