"""Dense SwiGLU feed-forward: down( silu(gate(x)) * up(x) ), no bias.

crates/cuda/src/engine.rs:4288-4303; silu(g) = g / (1 + exp(-g))
(crates/cuda/kernels/dense_kernels.cu:202-213). gate and up are one product:
their rows are interleaved in runs of 8 at load (8 gate rows, the 8 up rows of
the same features, ...), so that for few tokens the product's epilogue applies
the gate itself and for many the gate kernel reads both from one cache line.
A width that is no multiple of 8 keeps [gate; up] and the separate gate kernel.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import kernels
from ..config.schema import FeedForwardSpec
from ..weights import ParamDecl
from .base import NormTarget, split_input
from .registry import register_feed_forward


@register_feed_forward("swiglu")
class SwiGLU:
    graph_safe = True       # no host-side state: a decode step with it can be captured
    adds_in_place = True    # forward(..., resid=) may add the down projection into the stream
    takes_row_scaled = True     # x may be RowScaled: the gate/up product applies the row factor
    emits_for_norm = True       # forward(..., emit=) may fill a NormTarget from the down projection

    @classmethod
    def declare_params(cls, spec: FeedForwardSpec, prefix: str) -> List[ParamDecl]:
        return [ParamDecl(prefix + "gate_proj.weight", (spec.intermediate, spec.hidden)),
                ParamDecl(prefix + "up_proj.weight", (spec.intermediate, spec.hidden)),
                ParamDecl(prefix + "down_proj.weight", (spec.hidden, spec.intermediate))]

    def __init__(self, spec: FeedForwardSpec, weights: Dict[str, torch.Tensor], prefix: str,
                 dtype: torch.dtype, device: torch.device):
        self.spec = spec
        self.dtype = dtype
        gate, up = weights[prefix + "gate_proj.weight"], weights[prefix + "up_proj.weight"]
        I, h = spec.intermediate, spec.hidden
        self.group = getattr(kernels.current(), "GATE_GROUP", 0)
        if self.group and I % self.group == 0:
            g = self.group
            self.w_gate_up = torch.stack([gate.view(I // g, g, h), up.view(I // g, g, h)], dim=1) \
                .reshape(2 * I, h).contiguous()
        else:
            self.group = 0
            self.w_gate_up = torch.cat([gate, up], dim=0).contiguous()
        self.w_down = weights[prefix + "down_proj.weight"]

    def forward(self, x, batch, resid: Optional[torch.Tensor] = None, emit: Optional[NormTarget] = None):
        ops = kernels.current()
        x, row_sums = split_input(x)
        T = x.shape[0]
        I = self.spec.intermediate
        act = torch.empty((T, I), dtype=self.dtype, device=x.device)
        if self.group:
            if row_sums is None:
                ops.gated_linear(x, self.w_gate_up, act)
            else:
                ops.gated_linear(x, self.w_gate_up, act, row_sums=row_sums)
        else:
            gu = torch.empty((T, 2 * I), dtype=self.dtype, device=x.device)
            if row_sums is None:
                ops.linear(x, self.w_gate_up, gu)
            else:
                ops.linear_skinny(x, self.w_gate_up, gu, row_sums=row_sums)
            ops.silu_mul(gu, act)
        can_add = getattr(ops, "can_accumulate", None)
        if resid is not None and can_add and can_add(act, self.w_down):
            # x += act . Wd^T in the epilogue, which can also prepare the norm that follows
            if emit is not None and emit.finished:
                done = ops.linear_skinny(act, self.w_down, resid, accumulate=True, finish=emit.finish)
                return emit if done else None
            if emit is not None:
                written = ops.linear_skinny(act, self.w_down, resid, accumulate=True, emit=emit.emit)
                emit.ss = emit.ss[:written]          # as many partial sums a row as the kernel that ran has workgroups
                return emit
            ops.linear_skinny(act, self.w_down, resid, accumulate=True)
            return None
        out = torch.empty((T, self.spec.hidden), dtype=self.dtype, device=x.device)
        ops.linear(act, self.w_down, out)
        return out
