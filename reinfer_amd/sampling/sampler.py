"""Sampling on the GPU from the step's float32 logits.

Greedy takes the first maximum. Temperature > 0 draws by Gumbel-max with noise
that is a pure function of (request seed, position, token id), so a request
gets the same tokens whatever else is in the batch, however its prompt was cut
and whether or not it was preempted and recomputed
(crates/scheduler/src/rng.rs:52-66; crates/cuda/kernels/sampler_kernel.cu:61-77).
Filters and penalties, if asked for, mask or shift the logits first, in the
reference's order: repeat, frequency/presence, top-k, top-p, min-p, then
temperature and the draw (crates/samplers/src/lib.rs:66-90).
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from .. import kernels
from .params import SamplingParams

_MASK63 = (1 << 63) - 1


class SamplingError(RuntimeError):
    """No token could be drawn: every logit of a row is non-finite
    (bin/reinfer/src/pipeline.rs:189-191 raises on all-NaN logits)."""


def derive_seed(engine_seed: int, arrival: int) -> int:
    """Seed of a request that brings none: splitmix64(engine seed ^ arrival number)
    (bin/reinfer/src/sched_loop.rs:651-653)."""
    from ..weights.random_init import splitmix64
    return splitmix64((engine_seed ^ arrival) & ((1 << 64) - 1))


def as_int64(seed: int) -> int:
    seed &= (1 << 64) - 1
    return seed - (1 << 64) if seed >= (1 << 63) else seed


class Sampler:
    def __init__(self, device: torch.device):
        self.device = device

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams], seeds: Sequence[int],
               positions: Sequence[int], histories: Optional[Sequence[Sequence[int]]] = None) -> List[int]:
        """One token per row of ``logits``; ``positions[i]`` is the index the new
        token will have in its request, ``histories[i]`` the request's tokens so far."""
        n = logits.shape[0]
        if not (len(params) == len(seeds) == len(positions) == n):
            raise ValueError("one SamplingParams, seed and position per row")
        ops = kernels.current()
        if any(p.filters for p in params):
            if histories is None:
                raise ValueError("penalties need the requests' tokens")
            logits = logits.clone()
            ops.filter_logits(logits, params, histories)
        temp = torch.tensor([max(0.0, float(p.temperature)) for p in params], dtype=torch.float32)
        seeds_t = torch.tensor([as_int64(int(s)) for s in seeds], dtype=torch.int64)
        pos_t = torch.tensor([int(p) for p in positions], dtype=torch.int32)
        tokens = torch.empty(n, dtype=torch.int32, device=self.device)
        ops.sample(logits, temp.to(self.device), seeds_t.to(self.device), pos_t.to(self.device), tokens)
        out = tokens.tolist()
        for i, t in enumerate(out):
            if t < 0:
                raise SamplingError(f"row {i}: no finite logit to sample from")
        return out
