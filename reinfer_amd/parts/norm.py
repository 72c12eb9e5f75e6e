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

    def add_norm(self, resid: torch.Tensor, delta: Optional[torch.Tensor],
                 rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``resid += delta`` (float, in place) and the norm of the sum.

        With ``rows``, only those rows are computed, into a compact result, and
        the residual is left as it is.
        """
        n = resid.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.size), dtype=self.dtype, device=resid.device)
        kernels.current().add_rmsnorm(resid, delta, self.weight, self.eps, out, rows)
        return out
