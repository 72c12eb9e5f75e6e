"""Registries of the parts a layer is put together from, one per kind of part.

A part class is registered under the name that a spec's ``kind`` field holds.
Every part class has

    declare_params(spec, prefix) -> list[ParamDecl]     (classmethod)
    __init__(spec, weights, prefix, dtype, device)

and the methods of its kind (see the base classes in this package). A part sees
its own spec and tensors only.
"""
from __future__ import annotations

from typing import Any, Callable, Dict

_REGISTRIES: Dict[str, Dict[str, Any]] = {"mixer": {}, "feed_forward": {}, "norm": {}, "position": {},
                                          "block": {}}


def _register(kind_of_part: str, name: str, cls: Any = None):
    def deco(c):
        _REGISTRIES[kind_of_part][name] = c
        return c
    return deco(cls) if cls is not None else deco


def register_mixer(name: str, cls: Any = None):
    return _register("mixer", name, cls)


def register_feed_forward(name: str, cls: Any = None):
    return _register("feed_forward", name, cls)


def register_norm(name: str, cls: Any = None):
    return _register("norm", name, cls)


def register_position(name: str, cls: Any = None):
    return _register("position", name, cls)


def register_block(name: str, cls: Any = None):
    return _register("block", name, cls)


def lookup(kind_of_part: str, name: str):
    try:
        return _REGISTRIES[kind_of_part][name]
    except KeyError:
        known = sorted(_REGISTRIES[kind_of_part])
        raise KeyError(f"no {kind_of_part} part named {name!r}; registered: {known}") from None
