"""The kernels the parts call.

``current()`` returns the kernel set in use: the gfx950 library, loaded at first
use. There is no CPU or library fallback; without a GPU or without the built
library the first call raises. ``use()`` swaps the set for a block of code; the
CPU tests of the engine's bookkeeping put a stand-in there.
"""
from __future__ import annotations

import contextlib
from typing import Any, Optional

from .library import KernelLibraryError

_current: Optional[Any] = None


def current():
    global _current
    if _current is None:
        from .ops import HipKernels
        _current = HipKernels()
    return _current


@contextlib.contextmanager
def use(kernel_set):
    """Run a block with another kernel set (same method names as HipKernels)."""
    global _current
    prev = _current
    _current = kernel_set
    try:
        yield kernel_set
    finally:
        _current = prev


__all__ = ["KernelLibraryError", "current", "use"]
