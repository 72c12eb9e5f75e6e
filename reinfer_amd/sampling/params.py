"""Sampling options, with the reference's names and meanings
(crates/samplers/src/lib.rs:19-50; CLI flags bin/reinfer/src/main.rs:255-277)."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0            # <= 0: greedy, no randomness drawn
    top_k: Optional[int] = None         # keep the k most likely (None or 0: off)
    top_p: Optional[float] = None       # nucleus (None, <= 0 or >= 1: off)
    min_p: Optional[float] = None       # keep p >= min_p * max p
    repeat_penalty: Optional[float] = None      # > 1 to act: logit > 0 divided, < 0 multiplied
    frequency_penalty: Optional[float] = None   # logit -= count * penalty
    presence_penalty: Optional[float] = None    # logit -= penalty if seen
    repeat_last_n: int = 64             # penalties look at the last n tokens
    logit_bias: Tuple[Tuple[int, float], ...] = ()      # (token id, addend to its logit), each id once
    seed: Optional[int] = None          # None: derived from the engine's seed and the arrival number
    max_tokens: int = 256               # hard cap on generated tokens
    stop_token_ids: Tuple[int, ...] = ()        # beside the model's own end-of-sequence ids
    stop_sequences: Tuple[Tuple[int, ...], ...] = ()    # token sequences that end the request when generated
    ignore_eos: bool = False

    def __post_init__(self):
        if self.max_tokens < 1:
            raise ValueError("max_tokens must be at least 1")
        if self.temperature != self.temperature:
            raise ValueError("temperature is NaN")
        if self.top_k is not None and self.top_k < 0:
            raise ValueError("top_k must be >= 0")
        if self.top_p is not None and not self.top_p == self.top_p:
            raise ValueError("top_p is NaN")
        if self.repeat_last_n < 0:
            raise ValueError("repeat_last_n must be >= 0")
        # pairs (id, bias), each id once (the reference looks an id up in its sorted list,
        # crates/cuda/src/sampler.rs:235; crates/cuda/kernels/sampler_kernel.cu:195-203)
        pairs = tuple((int(t), float(b)) for t, b in
                      (self.logit_bias.items() if isinstance(self.logit_bias, dict) else self.logit_bias))
        if len({t for t, _ in pairs}) != len(pairs):
            raise ValueError("logit_bias names a token id twice")
        if any(t < 0 for t, _ in pairs) or any(b != b for _, b in pairs):
            raise ValueError("logit_bias: token ids are >= 0 and biases are numbers")
        object.__setattr__(self, "logit_bias", tuple(sorted(pairs)))
        # stop strings arrive as token-id sequences (the text belongs to the layer above,
        # crates/scheduler/src/stop.rs:1-6); empty ones are ignored
        object.__setattr__(self, "stop_sequences",
                           tuple(tuple(int(t) for t in seq) for seq in self.stop_sequences if len(seq) > 0))

    @property
    def greedy(self) -> bool:
        return self.temperature <= 0.0

    @property
    def filters(self) -> bool:
        """True if anything beside temperature shapes the distribution."""
        return bool((self.top_k or 0) > 0 or (self.top_p is not None and 0.0 < self.top_p < 1.0)
                    or (self.min_p or 0.0) > 0.0 or self.penalties or len(self.logit_bias) > 0)

    @property
    def penalties(self) -> bool:
        return bool((self.repeat_penalty or 0.0) > 1.0 or (self.frequency_penalty or 0.0) > 0.0
                    or (self.presence_penalty or 0.0) > 0.0)
