"""Position encodings. A mixer holds one and passes its constants to its kernel.

Rotation: pair (j, j + R/2) ("rope_neox", half split) or (2j, 2j + 1)
("rope_interleaved") is turned by the angle pos * theta^(-2j/R)
(crates/cuda/kernels/dense_kernels.cu:125-139; crates/kernels/src/refs.rs:25-37).
The reference computes theta^(-2j/R) with powf in the kernel; here the table of
R/2 inverse frequencies is made once, in double precision, and rounded to float.
The angle itself (position times frequency) and its sine and cosine are float.
"""
from __future__ import annotations

from typing import List

import torch

from ..config.schema import PositionSpec
from .registry import register_position


class _Rotary:
    style = 0

    def __init__(self, spec: PositionSpec, device: torch.device):
        if spec.rotary_dim <= 0 or spec.rotary_dim % 2 != 0:
            raise ValueError(f"rotation needs an even, positive width, got {spec.rotary_dim}")
        self.rotary_dim = spec.rotary_dim
        self.theta = float(spec.theta)
        j = torch.arange(spec.rotary_dim // 2, dtype=torch.float64)
        inv = torch.pow(torch.tensor(self.theta, dtype=torch.float64), -2.0 * j / spec.rotary_dim)
        self.inv_freq = inv.to(torch.float32).to(device)


@register_position("rope_neox")
class RotaryHalfSplit(_Rotary):
    style = 0


@register_position("rope_interleaved")
class RotaryInterleaved(_Rotary):
    style = 1


@register_position("none")
class NoPosition:
    style = 0
    rotary_dim = 0

    def __init__(self, spec: PositionSpec, device: torch.device):
        self.inv_freq = torch.zeros(1, dtype=torch.float32, device=device)
