"""Grouped-query attention over the paged cache.

q/k/v projections (one fused product), optional per-head RMSNorm of q and k,
rotation, cache write, attention over the request's block table, output
projection. Order and formulas: crates/cuda/src/engine.rs:4090-4281 (decode) and
:5462-5621 (whole prompt); the reference has separate kernels for head norm,
rotation, scale and cache write and separate calls for prompts and decoding,
here one fused kernel and one call serve any mix of both. The scale multiplies
the float score, not q (the reference scales and re-rounds q, engine.rs:4150-4160).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import kernels
from ..config.schema import MixerSpec
from ..weights import MATRIX, VECTOR, ParamDecl
from .base import KVNeed, LayerCache, NormTarget, split_input
from .registry import lookup, register_mixer


@register_mixer("gqa_attention")
class GroupedQueryAttention:
    graph_safe = True       # no host-side state: a decode step with it can be captured
    adds_in_place = True    # forward(..., resid=) may add the output projection into the stream
    takes_row_scaled = True     # x may be RowScaled: the q/k/v product applies the row factor
    emits_for_norm = True       # forward(..., emit=) may fill a NormTarget from the output projection

    @classmethod
    def declare_params(cls, spec: MixerSpec, prefix: str) -> List[ParamDecl]:
        nq = spec.num_heads * spec.head_dim
        nkv = spec.num_kv_heads * spec.head_dim
        out = [ParamDecl(prefix + "q_proj.weight", (nq, spec.hidden)),
               ParamDecl(prefix + "k_proj.weight", (nkv, spec.hidden)),
               ParamDecl(prefix + "v_proj.weight", (nkv, spec.hidden)),
               ParamDecl(prefix + "o_proj.weight", (spec.hidden, nq))]
        if spec.bias:
            out += [ParamDecl(prefix + "q_proj.bias", (nq,), init="zeros", role=MATRIX),
                    ParamDecl(prefix + "k_proj.bias", (nkv,), init="zeros", role=MATRIX),
                    ParamDecl(prefix + "v_proj.bias", (nkv,), init="zeros", role=MATRIX)]
        if spec.qk_norm:
            out += [ParamDecl(prefix + "q_norm.weight", (spec.head_dim,), init="norm", role=VECTOR),
                    ParamDecl(prefix + "k_norm.weight", (spec.head_dim,), init="norm", role=VECTOR)]
        return out

    def __init__(self, spec: MixerSpec, weights: Dict[str, torch.Tensor], prefix: str,
                 dtype: torch.dtype, device: torch.device):
        if spec.num_heads <= 0 or spec.num_kv_heads <= 0 or spec.num_heads % spec.num_kv_heads:
            raise ValueError(f"{spec.num_heads} query heads do not divide into {spec.num_kv_heads} groups")
        self.spec = spec
        self.dtype = dtype
        self.num_heads, self.num_kv_heads, self.head_dim = spec.num_heads, spec.num_kv_heads, spec.head_dim
        self.scale = float(spec.scale)
        self.window = int(spec.window)
        self.qkv_width = (spec.num_heads + 2 * spec.num_kv_heads) * spec.head_dim
        # rows of q, k, v one after the other: stays [out, in], K contiguous
        self.w_qkv = torch.cat([weights[prefix + "q_proj.weight"], weights[prefix + "k_proj.weight"],
                                weights[prefix + "v_proj.weight"]], dim=0).contiguous()
        self.b_qkv = None
        if spec.bias:
            self.b_qkv = torch.cat([weights[prefix + "q_proj.bias"], weights[prefix + "k_proj.bias"],
                                    weights[prefix + "v_proj.bias"]], dim=0).to(dtype).contiguous()
        self.w_o = weights[prefix + "o_proj.weight"]
        self.q_norm = weights[prefix + "q_norm.weight"] if spec.qk_norm else None
        self.k_norm = weights[prefix + "k_norm.weight"] if spec.qk_norm else None
        self.eps = float(spec.qk_norm_eps)
        self.position = lookup("position", spec.position.kind)(spec.position, device)
        if self.position.rotary_dim > spec.head_dim:
            raise ValueError("the rotated width cannot exceed the head size")

    def cache_need(self) -> KVNeed:
        return KVNeed(self.num_kv_heads, self.head_dim, self.window)

    def plan_captured_step(self, batch, num_rows: int, ctx_cap: int) -> None:
        # the attention kernels pick their grids by host-side numbers of the step: the kernel set fixes them
        hook = getattr(kernels.current(), "plan_captured_step", None)
        if hook is not None:
            hook(batch, num_rows, ctx_cap)

    def forward(self, x, batch, cache: LayerCache, resid: Optional[torch.Tensor] = None,
                emit: Optional[NormTarget] = None):
        ops = kernels.current()
        x, row_sums = split_input(x)
        T = x.shape[0]
        slots = batch.slots[cache.group] if cache.writes else batch.no_slots
        # a product that the kernels cut into K ranges may hand them over unadded: the kernel behind it
        # adds them as it reads, which saves the adding kernel (and applies a carried norm's row factor)
        in_ranges = getattr(ops, "linear_ranges", None)
        ranges = in_ranges(x, self.w_qkv) if in_ranges is not None and self.b_qkv is None else None
        if ranges is not None:
            q_rows, q_stride = torch.empty((T, self.num_heads * self.head_dim), dtype=self.dtype, device=x.device), \
                self.num_heads * self.head_dim
            ops.qk_norm_rope_cache_ranges(ranges, row_sums, q_rows, self.q_norm, self.k_norm, self.eps,
                                          batch.positions, self.position.inv_freq, self.position.rotary_dim,
                                          self.position.style, slots, cache.k, cache.v, self.num_heads,
                                          self.num_kv_heads, self.head_dim)
        else:
            q_rows, q_stride = torch.empty((T, self.qkv_width), dtype=self.dtype, device=x.device), self.qkv_width
            if row_sums is None:
                ops.linear(x, self.w_qkv, q_rows, self.b_qkv)
            else:
                ops.linear_skinny(x, self.w_qkv, q_rows, self.b_qkv, row_sums=row_sums)
            ops.qk_norm_rope_cache(q_rows, self.q_norm, self.k_norm, self.eps, batch.positions,
                                   self.position.inv_freq, self.position.rotary_dim, self.position.style,
                                   slots, cache.k, cache.v, self.num_heads, self.num_kv_heads, self.head_dim)
        attn = torch.empty((T, self.num_heads * self.head_dim), dtype=self.dtype, device=x.device)
        ops.attention(q_rows, q_stride, attn, cache.k, cache.v, batch, self.num_heads,
                      self.num_kv_heads, self.head_dim, self.scale, self.window, cache.group)
        can_add = getattr(ops, "can_accumulate", None)
        if resid is not None and can_add and can_add(attn, self.w_o):
            # x += attn . Wo^T in the epilogue, which can also prepare the norm that follows
            if emit is not None and emit.finished:
                done = ops.linear_skinny(attn, self.w_o, resid, accumulate=True, finish=emit.finish)
                return emit if done else None
            if emit is not None:
                written = ops.linear_skinny(attn, self.w_o, resid, accumulate=True, emit=emit.emit)
                emit.ss = emit.ss[:written]          # as many partial sums a row as the kernel that ran has workgroups
                return emit
            ops.linear_skinny(attn, self.w_o, resid, accumulate=True)
            return None
        out = torch.empty((T, self.spec.hidden), dtype=self.dtype, device=x.device)
        ops.linear(attn, self.w_o, out)
        return out
