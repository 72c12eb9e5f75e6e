"""Binding tensors of a model folder to the parameters the parts declare.

Every part lists what it needs as :class:`ParamDecl` (full tensor name, shape,
how a random model initialises it, and whether it is a matrix, a vector or an
integer table). The loader reads ``model.safetensors`` (or the shards named by
``model.safetensors.index.json``), checks all names and shapes and raises ONE
:class:`WeightError` that lists everything wrong. The reference checks rank and
exact shape per tensor and fails on the first (crates/cuda/src/engine.rs:3213-3238).

Storage: floating matrices are kept in the compute dtype (bfloat16 for serving,
float32 for the 32-bit path). Vectors that the file stores in 32-bit stay in
32-bit also under bfloat16; integer tables are int32.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Dict, Iterable, List, Mapping, Optional, Sequence, Tuple

import torch

from .safetensors_io import SafetensorsError, SafetensorsFile

MATRIX = "matrix"
VECTOR = "vector"
INT_TABLE = "int_table"


@dataclass(frozen=True)
class ParamDecl:
    name: str
    shape: Tuple[int, ...]
    init: str = "normal"        # "normal": N(0, 0.02); "norm": U(0.8, 1.2); "zeros"; "int"
    role: str = MATRIX
    optional: bool = False      # absent is fine (e.g. a head that is tied)


class WeightError(ValueError):
    """Names that are missing or unexpected and tensors of the wrong shape, all at once."""

    def __init__(self, where: str, missing: Sequence[str], unexpected: Sequence[str],
                 wrong_shape: Sequence[Tuple[str, Tuple[int, ...], Tuple[int, ...]]],
                 wrong_dtype: Sequence[Tuple[str, str]] = ()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_dtype = list(wrong_dtype)
        lines = [f"{where}: weights do not match the model"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, want, got in self.wrong_shape:
            lines.append(f"  wrong shape: {name}: expected {list(want)} got {list(got)}")
        for name, tag in self.wrong_dtype:
            lines.append(f"  unsupported dtype: {name}: {tag}")
        super().__init__("\n".join(lines))


def storage_dtype(decl: ParamDecl, stored: torch.dtype, compute: torch.dtype) -> torch.dtype:
    if decl.role == INT_TABLE:
        return torch.int32
    if compute == torch.float32:
        return torch.float32
    if decl.role == VECTOR and stored == torch.float32:
        return torch.float32
    return compute


# names some exporters add that carry no parameter of the model
_IGNORABLE_SUFFIXES = ("rotary_emb.inv_freq",)


def _open_folder(model_dir: str) -> Tuple[Dict[str, SafetensorsFile], Dict[str, str]]:
    """-> (open files by file name, tensor name -> file name)."""
    single = os.path.join(model_dir, "model.safetensors")
    index = os.path.join(model_dir, "model.safetensors.index.json")
    files: Dict[str, SafetensorsFile] = {}
    where: Dict[str, str] = {}
    if os.path.isfile(single):
        files["model.safetensors"] = SafetensorsFile(single)
        for n in files["model.safetensors"].names():
            where[n] = "model.safetensors"
    elif os.path.isfile(index):
        with open(index, "r", encoding="utf-8") as f:
            wm = json.load(f).get("weight_map", {})
        for name, fname in wm.items():
            if fname not in files:
                files[fname] = SafetensorsFile(os.path.join(model_dir, fname))
            where[name] = fname
    else:
        raise FileNotFoundError(f"{model_dir}: neither model.safetensors nor model.safetensors.index.json")
    return files, where


def load_weights(model_dir: str, decls: Sequence[ParamDecl], compute_dtype: torch.dtype,
                 device: torch.device, allow_unexpected: bool = False,
                 report: Optional[Dict[str, object]] = None) -> Dict[str, torch.Tensor]:
    """Tensors that no part declares are an error like the others (a folder that holds another model's
    tensors is more often a mistake than an exporter's extras); with ``allow_unexpected`` they are
    left unread, as the reference leaves what it does not ask for (crates/cuda/src/engine.rs:3216-3235),
    and ``report["unexpected"]`` lists them."""
    files, where = _open_folder(model_dir)
    try:
        wanted = {d.name: d for d in decls}
        missing = [d.name for d in decls if d.name not in where and not d.optional]
        unexpected = [n for n in where if n not in wanted and not n.endswith(_IGNORABLE_SUFFIXES)]
        if report is not None:
            report["unexpected"] = list(unexpected)
        if allow_unexpected:
            unexpected = []
        wrong_shape, wrong_dtype = [], []
        for d in decls:
            if d.name not in where:
                continue
            f = files[where[d.name]]
            if d.name not in f.entries:
                missing.append(d.name)
                continue
            got = f.shape(d.name)
            if tuple(got) != tuple(d.shape):
                wrong_shape.append((d.name, tuple(d.shape), tuple(got)))
            tag = f.dtype_tag(d.name)
            ok = ("I64", "I32", "I16", "I8", "U8") if d.role == INT_TABLE else ("F32", "F16", "BF16")
            if tag not in ok:
                wrong_dtype.append((d.name, tag))
        if missing or unexpected or wrong_shape or wrong_dtype:
            raise WeightError(model_dir, missing, unexpected, wrong_shape, wrong_dtype)
        out: Dict[str, torch.Tensor] = {}
        for d in decls:
            if d.name not in where:
                continue
            t = files[where[d.name]].tensor(d.name)
            out[d.name] = t.to(storage_dtype(d, t.dtype, compute_dtype)).to(device)
        return out
    finally:
        for f in files.values():
            f.close()


def weight_from_folder(model_dir: str, name: str) -> torch.Tensor:
    """One tensor of a model folder, as stored, on the CPU."""
    files, where = _open_folder(model_dir)
    try:
        if name not in where:
            raise KeyError(f"{model_dir}: no tensor {name}")
        return files[where[name]].tensor(name).clone()
    finally:
        for f in files.values():
            f.close()


def check_tensors(where: str, decls: Sequence[ParamDecl], tensors: Mapping[str, torch.Tensor]) -> None:
    """The same one-error check for tensors handed over in memory."""
    wanted = {d.name: d for d in decls}
    missing = [d.name for d in decls if d.name not in tensors and not d.optional]
    unexpected = [n for n in tensors if n not in wanted]
    wrong = [(d.name, tuple(d.shape), tuple(tensors[d.name].shape)) for d in decls
             if d.name in tensors and tuple(tensors[d.name].shape) != tuple(d.shape)]
    if missing or unexpected or wrong:
        raise WeightError(where, missing, unexpected, wrong)
