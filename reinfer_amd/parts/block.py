"""How norm, mixer and feed-forward are arranged in a layer.

"prenorm": x += mixer(norm(x)); x += ffn(norm(x))
(crates/cuda/src/engine.rs:4075-4314). The residual stream is float. A block
gets the stream and the previous block's last addend, not yet added, so that
the add and the norm are one kernel (the reference fuses the same pair for the
o-projection, dense_kernels.cu:257-274); it returns its own last addend, or
None if its last part added it into the stream itself.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..config.schema import BlockSpec
from ..weights import ParamDecl
from .base import LayerCache
from .registry import lookup, register_block


@register_block("prenorm")
class PreNormBlock:
    @classmethod
    def declare_params(cls, spec: BlockSpec) -> List[ParamDecl]:
        p = spec.prefix
        out = lookup("norm", spec.mixer_norm.kind).declare_params(spec.mixer_norm, p + spec.mixer_norm_name)
        out += lookup("mixer", spec.mixer.kind).declare_params(spec.mixer, p + spec.mixer_prefix)
        out += lookup("norm", spec.ffn_norm.kind).declare_params(spec.ffn_norm, p + spec.ffn_norm_name)
        out += lookup("feed_forward", spec.ffn.kind).declare_params(spec.ffn, p + spec.ffn_prefix)
        return out

    def __init__(self, spec: BlockSpec, weights: Dict[str, torch.Tensor], dtype: torch.dtype,
                 device: torch.device):
        missing = [n for n in ("mixer", "ffn", "mixer_norm", "ffn_norm") if getattr(spec, n) is None]
        if missing:
            raise ValueError(f"a prenorm block is made of a mixer, a feed-forward and a norm before each; "
                             f"block {spec.prefix!r} names no {', '.join(missing)}")
        p = spec.prefix
        self.spec = spec
        self.mixer_norm = lookup("norm", spec.mixer_norm.kind)(spec.mixer_norm, weights,
                                                               p + spec.mixer_norm_name, dtype, device)
        self.mixer = lookup("mixer", spec.mixer.kind)(spec.mixer, weights, p + spec.mixer_prefix, dtype, device)
        self.ffn_norm = lookup("norm", spec.ffn_norm.kind)(spec.ffn_norm, weights,
                                                           p + spec.ffn_norm_name, dtype, device)
        self.ffn = lookup("feed_forward", spec.ffn.kind)(spec.ffn, weights, p + spec.ffn_prefix, dtype, device)

    passes_emit = True      # forward(..., emit=) hands a NormTarget on to the feed-forward

    def cache_need(self):
        """What this layer keeps between steps: its mixer's need."""
        return self.mixer.cache_need() if hasattr(self.mixer, "cache_need") else None

    def parts(self):
        """The parts this arrangement is made of (for whoever asks every part something)."""
        return (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn)

    def entry_target(self, resid: torch.Tensor):
        """A NormTarget for this block's first norm, for the part that runs before the block, or
        None if the norm or the mixer behind it cannot use one."""
        if not hasattr(self.mixer_norm, "emit_target"):
            return None
        return self.mixer_norm.emit_target(resid, getattr(self.mixer, "takes_row_scaled", False))

    def forward(self, resid: torch.Tensor, delta, batch, cache: Optional[LayerCache], emit=None):
        # A part that declares ``adds_in_place`` also gets the residual stream: where its last
        # product can add into it, it does and returns None; any other part returns its addend.
        # Where that product can also prepare the norm that follows (the part ``emits_for_norm``,
        # the norm offers a target, and the part behind the norm ``takes_row_scaled``), the norm
        # costs no kernel: its column weight is applied by the product before it, its row
        # factor by the product after it.
        mixer, ffn = self.mixer, self.ffn
        xn = self._norm(self.mixer_norm, resid, delta, mixer)
        if getattr(mixer, "adds_in_place", False):
            tgt = self._target(self.ffn_norm, resid, mixer, ffn)
            if tgt is not None:
                a = mixer.forward(xn, batch, cache, resid=resid, emit=tgt)
            else:
                a = mixer.forward(xn, batch, cache, resid=resid)
        else:
            a = mixer.forward(xn, batch, cache)
        xn = self._norm(self.ffn_norm, resid, a, ffn)
        if getattr(ffn, "adds_in_place", False):
            if emit is not None and getattr(ffn, "emits_for_norm", False):
                return ffn.forward(xn, batch, resid=resid, emit=emit)
            return ffn.forward(xn, batch, resid=resid)
        return ffn.forward(xn, batch)

    @staticmethod
    def _norm(norm, resid, delta, consumer):
        if hasattr(norm, "emit_target"):
            return norm.add_norm(resid, delta, scaled_ok=getattr(consumer, "takes_row_scaled", False))
        if not isinstance(delta, torch.Tensor) and delta is not None:
            delta = None               # a filled target: the sum is already in the stream
        return norm.add_norm(resid, delta)

    @staticmethod
    def _target(norm, resid, producer, consumer):
        if not (getattr(producer, "emits_for_norm", False) and hasattr(norm, "emit_target")):
            return None
        return norm.emit_target(resid, getattr(consumer, "takes_row_scaled", False))
