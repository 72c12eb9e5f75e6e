"""RMSNorm, alone and fused with the residual add.

y = x * rsqrt(mean(x^2) + eps) * w, eps inside the root
(crates/cuda/kernels/dense_kernels.cu:59-88; crates/kernels/src/refs.rs:10-18).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import kernels
from ..config.schema import NormSpec
from ..weights import VECTOR, ParamDecl
from .base import NormTarget, RowScaled
from .registry import register_norm


@register_norm("rmsnorm")
class RMSNorm:
    @classmethod
    def declare_params(cls, spec: NormSpec, name: str) -> List[ParamDecl]:
        return [ParamDecl(name, (spec.size,), init="norm", role=VECTOR)]

    def __init__(self, spec: NormSpec, weights: Dict[str, torch.Tensor], name: str,
                 dtype: torch.dtype, device: torch.device):
        self.size = spec.size
        self.eps = float(spec.eps)
        self.weight = weights[name]
        self.dtype = dtype

    def add_norm(self, resid: torch.Tensor, delta, rows: Optional[torch.Tensor] = None,
                 scaled_ok: bool = False):
        """``resid += delta`` (float, in place) and the norm of the sum.

        With ``rows``, only those rows are computed, into a compact result, and
        the residual is left as it is. ``delta`` may be None (nothing to add) or a
        :class:`NormTarget` that the previous part filled for this norm: the sum is
        in the stream already, and if the caller takes :class:`RowScaled`
        (``scaled_ok``) there is nothing left to launch.
        """
        if isinstance(delta, NormTarget):
            if delta.norm is self and rows is None:
                if delta.finished:
                    return delta.x             # the product before wrote the finished rows
                if scaled_ok:
                    return RowScaled(delta.x, delta.ss, self.eps, self.size)
            delta = None
        n = resid.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.size), dtype=self.dtype, device=resid.device)
        kernels.current().add_rmsnorm(resid, delta, self.weight, self.eps, out, rows)
        return out

    def emit_target(self, resid: torch.Tensor, consumer_scales: bool = True) -> Optional[NormTarget]:
        """Buffers for a part that adds into ``resid`` with a product that can also prepare this
        norm (bfloat16, few rows); None where that does not apply. Up to the rows of the weight-streaming
        products, and where the part behind the norm applies a row factor (``consumer_scales``), the half-done
        form; for the rows above them that the adding kernel can still finish, the finished form."""
        ops = kernels.current()
        parts = getattr(ops, "skinny_row_parts", None)
        T = resid.shape[0]
        # the product behind this norm reads rows of this width as 16-byte pieces: a width that is no
        # multiple of 8 goes through the norm kernel and the plain product
        if parts is None or self.dtype != torch.bfloat16 or resid.shape[1] != self.size or self.size % 8 != 0:
            return None
        few = getattr(ops, "NORM_ON_PRODUCTS_ROWS", 0)
        if few < T <= getattr(ops, "NORM_FINISHED_ROWS", 0):
            return NormTarget(self, torch.empty((T, self.size), dtype=torch.bfloat16, device=resid.device), None,
                              finished=True)
        if T > few or not consumer_scales:
            return None
        return NormTarget(self,
                          torch.empty((T, self.size), dtype=torch.bfloat16, device=resid.device),
                          torch.empty((parts(T, self.size), T), dtype=torch.float32, device=resid.device))
