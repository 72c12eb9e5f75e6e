"""Loads the host runtime (``reinfer_amd._host``, C++ with pybind11): paged-cache
bookkeeping, packing of a step's index arrays, and the scheduler. It is built
in-tree at first use if it is not there (or into the temporary folder when the
tree cannot be written). The exceptions it raises are defined here, in Python,
so that they can carry attributes.
"""
from __future__ import annotations

import importlib.util
import sys


class OutOfBlocks(RuntimeError):
    """A pool cannot give the blocks asked for (crates/memory/src/pool.rs OutOfPages{need, free})."""

    def __init__(self, group: int, need: int, free: int):
        super().__init__(f"cache group {group}: need {need} blocks, {free} free")
        self.group, self.need, self.free = group, need, free


class OutOfSlots(RuntimeError):
    pass


class RequestRefused(ValueError):
    pass


class StepError(ValueError):
    """A step was asked for something it cannot run (checked before any launch);
    the reference's step checks the same on the host (crates/cuda/src/engine.rs:5854-5943)."""


def _load():
    name = "reinfer_amd._host"
    if name in sys.modules:
        return sys.modules[name]
    from .csrc import build
    path = build.ensure_host_built()
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    mod.set_exceptions(OutOfBlocks, OutOfSlots, RequestRefused, StepError)
    sys.modules[name] = mod
    return mod


host = _load()
