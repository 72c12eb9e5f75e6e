"""Per-kernel-class GPU time of a step, measured with events around every call
into the kernel set.

    timed = TimedKernels(kernels.current())
    timed.name_weight(block.mixer.w_qkv, "qkv")          # products are classed by their weight
    with kernels.use(timed):
        timed.hold_back(20.0)                            # the GPU busy elsewhere while the step is queued
        runner.step(entries)
    rows = timed.report()                                # class -> calls, milliseconds

The reference brackets the segments of its decode step the same way, with
events on the stream (crates/cuda/src/engine.rs:1146-1408) and prints them with
``--perf`` (bin/reinfer/src/main.rs:706-727). Two things make the figures mean
what a captured step costs: the step is queued behind work that keeps the GPU
busy meanwhile (``hold_back``), so that no kernel waits for the host between
its two events; and an event pair costs the stream about a microsecond, which
``report`` measures on an empty pair and takes off every class.
"""
from __future__ import annotations

from typing import Any, Callable, Dict, List, Optional, Tuple

import torch

# methods of the kernel set that launch work, and how their calls are classed
_ROWS = {"embed": "embedding", "add_rmsnorm": "norm", "silu_mul": "gate", "sample": "sampler",
         "filter_logits": "sampler"}
_QK = {"qk_norm_rope_cache", "qk_norm_rope_cache_ranges"}
_ATTN = {"attention", "attention_plain", "attention_decode", "attention_prefill"}
_LINEAR = {"linear", "linear_plain", "linear_skinny", "gated_linear", "linear_ranges"}


class TimedKernels:
    """A kernel set that times every call of the set it wraps."""

    def __init__(self, inner):
        self._inner = inner
        self._names: Dict[int, str] = {}
        self._spans: List[Tuple[str, torch.cuda.Event, torch.cuda.Event]] = []
        self._filler: Optional[torch.Tensor] = None
        self.name = getattr(inner, "name", "timed")

    def name_weight(self, weight: torch.Tensor, role: str) -> None:
        self._names[weight.data_ptr()] = role

    def _label(self, method: str, args, kwargs) -> str:
        if method in _ROWS:
            return _ROWS[method]
        if method in _QK:
            return "head norm + rotation + cache write"
        if method in _ATTN:
            return "attention"
        if method in _LINEAR:
            w = args[1] if len(args) > 1 else kwargs.get("weight")
            role = self._names.get(w.data_ptr()) if isinstance(w, torch.Tensor) else None
            return role or f"product {w.shape[0]}x{w.shape[1]}"
        return method

    def __getattr__(self, attr: str) -> Any:
        target = getattr(self._inner, attr)
        if not callable(target) or not (attr in _ROWS or attr in _QK or attr in _ATTN or attr in _LINEAR):
            return target

        def timed_call(*args, **kwargs):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            out = target(*args, **kwargs)
            e1.record()
            self._spans.append((self._label(attr, args, kwargs), e0, e1))
            return out
        return timed_call

    def hold_back(self, milliseconds: float, device="cuda:0") -> None:
        """Queue about this much reading of a large buffer, so that the host can queue a whole step
        behind it (the step's kernels then run back to back, as in a replayed graph)."""
        size = 2 << 30
        if self._filler is None:
            self._filler = torch.empty(size // 4, dtype=torch.int32, device=device).random_()
            self._sink = torch.zeros(1, dtype=torch.int32, device=device)
        from . import library
        reads = max(1, int(milliseconds / (size / 5.5e12 * 1e3)))
        for _ in range(reads):
            library.call("ra_stream_read", self._filler.data_ptr(), size, self._sink.data_ptr(),
                         torch.cuda.current_stream().cuda_stream)

    def report(self) -> Dict[str, Dict[str, float]]:
        """class -> {"calls", "ms"}; clears what was recorded."""
        pairs = []
        for _ in range(16):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            e1.record()
            pairs.append((e0, e1))
        torch.cuda.synchronize()
        empty = sorted(a.elapsed_time(b) for a, b in pairs)[len(pairs) // 2]
        out: Dict[str, Dict[str, float]] = {}
        for label, e0, e1 in self._spans:
            row = out.setdefault(label, {"calls": 0, "ms": 0.0})
            row["calls"] += 1
            row["ms"] += max(0.0, e0.elapsed_time(e1) - empty)
        self._spans = []
        return out
