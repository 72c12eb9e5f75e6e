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
        p = spec.prefix
        self.spec = spec
        self.mixer_norm = lookup("norm", spec.mixer_norm.kind)(spec.mixer_norm, weights,
                                                               p + spec.mixer_norm_name, dtype, device)
        self.mixer = lookup("mixer", spec.mixer.kind)(spec.mixer, weights, p + spec.mixer_prefix, dtype, device)
        self.ffn_norm = lookup("norm", spec.ffn_norm.kind)(spec.ffn_norm, weights,
                                                           p + spec.ffn_norm_name, dtype, device)
        self.ffn = lookup("feed_forward", spec.ffn.kind)(spec.ffn, weights, p + spec.ffn_prefix, dtype, device)

    def forward(self, resid: torch.Tensor, delta: Optional[torch.Tensor], batch,
                cache: Optional[LayerCache]) -> torch.Tensor:
        # A part that declares ``adds_in_place`` also gets the residual stream: where its last
        # product can add into it, it does and returns None; any other part returns its addend.
        xn = self.mixer_norm.add_norm(resid, delta)
        if getattr(self.mixer, "adds_in_place", False):
            a = self.mixer.forward(xn, batch, cache, resid=resid)
        else:
            a = self.mixer.forward(xn, batch, cache)
        xn = self.ffn_norm.add_norm(resid, a)
        if getattr(self.ffn, "adds_in_place", False):
            return self.ffn.forward(xn, batch, resid=resid)
        return self.ffn.forward(xn, batch)
