"""A decoder put together from a :class:`ModelSpec`: embedding, blocks in run
order, final norm, head. It knows no architecture by name; what differs between
architectures is in the spec and in the parts the spec names.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

from .. import kernels
from ..config.schema import ModelSpec
from ..parts import KVNeed, LayerCache, StateNeed, lookup
from ..weights import MATRIX, ParamDecl


def declare_params(spec: ModelSpec) -> List[ParamDecl]:
    """Every tensor the model reads, each once, in a fixed order."""
    out = [ParamDecl(spec.embed_name, (spec.vocab_size, spec.hidden))]
    if spec.input_position is not None:
        part = lookup("position", spec.input_position.kind)
        if hasattr(part, "declare_input_params"):
            out += part.declare_input_params(spec.input_position, spec.input_position_prefix)
    for b in spec.blocks:
        out += lookup("block", b.kind).declare_params(b)
    out += lookup("norm", spec.final_norm.kind).declare_params(spec.final_norm, spec.final_norm_name)
    # a tied model may still carry a head tensor in its file: it is not read
    out.append(ParamDecl(spec.head_name, (spec.vocab_size, spec.hidden), optional=spec.tie_embeddings))
    seen = set()
    for d in out:
        if d.name in seen:
            raise ValueError(f"tensor {d.name} is declared twice")
        seen.add(d.name)
    return out


class DecoderModel:
    def __init__(self, spec: ModelSpec, weights: Dict[str, torch.Tensor], dtype: torch.dtype,
                 device: torch.device):
        self.spec = spec
        self.dtype = dtype
        self.device = device
        self.embed = weights[spec.embed_name]
        # a position part at the embedding stage: built with the model's tensors, it adds its encoding of
        # the step's positions into the stream (``add_to_stream(resid, batch)``)
        self.input_position = None
        if spec.input_position is not None:
            part = lookup("position", spec.input_position.kind)
            if not hasattr(part, "add_to_stream"):
                raise ValueError(f"position part {spec.input_position.kind!r} cannot stand at the embedding: "
                                 "it has no add_to_stream(resid, batch)")
            self.input_position = part(spec.input_position, device, weights=weights,
                                       prefix=spec.input_position_prefix, dtype=dtype)
        self.blocks = [lookup("block", b.kind)(b, weights, dtype, device) for b in spec.blocks]
        self.final_norm = lookup("norm", spec.final_norm.kind)(spec.final_norm, weights,
                                                               spec.final_norm_name, dtype, device)
        # tied: the embedding matrix is the head (crates/cpu/src/model.rs:218-225)
        self.head = self.embed if spec.tie_embeddings else weights[spec.head_name]
        self.run_order = spec.run_order

    def cache_needs(self) -> List[Optional[object]]:
        """What each run-order entry keeps: KVNeed, PagedNeed, StateNeed, or None. The block arrangement
        answers (``cache_need()``); one that does not is asked for a ``mixer`` attribute's answer."""
        needs: List[Optional[object]] = []
        for e in self.run_order:
            block = self.blocks[e.block]
            if hasattr(block, "cache_need"):
                needs.append(block.cache_need())
                continue
            mixer = getattr(block, "mixer", None)
            needs.append(mixer.cache_need() if mixer is not None and hasattr(mixer, "cache_need") else None)
        return needs

    def parts(self):
        """Every part of the model once: blocks, what they say they are made of, the norms and position part
        at either end."""
        seen, out = set(), []
        def add(p):
            if p is not None and id(p) not in seen:
                seen.add(id(p))
                out.append(p)
        add(self.input_position)
        for b in self.blocks:
            add(b)
            for p in (b.parts() if hasattr(b, "parts") else (getattr(b, "mixer", None), getattr(b, "ffn", None))):
                add(p)
        add(self.final_norm)
        return out

    def plan_captured_step(self, batch, num_rows: int, ctx_cap: int) -> None:
        """A decode step that is captured once and replayed takes no host-side number from the step it
        replays for: whatever a part's kernels choose grids or buffers by on the host must be fixed for the
        bucket. Every part with a ``plan_captured_step(batch, num_rows, ctx_cap)`` is asked to write what it
        needs into ``batch.extra`` (``num_rows`` requests of one token each, contexts of at most ``ctx_cap``)."""
        for p in self.parts():
            hook = getattr(p, "plan_captured_step", None)
            if hook is not None:
                hook(batch, num_rows, ctx_cap)

    def forward_layers(self, batch, caches: Sequence[Optional[LayerCache]], observer=None):
        """Embedding and all blocks: (residual stream, last addend not yet added).

        ``observer(i, hidden)``, if given, is called with the float32 hidden state [T, hidden] behind
        the embedding (i = 0) and behind run-order entry i - 1 (the reference reads activations back
        layer by layer the same way, crates/cuda/src/engine.rs:3744-3765)."""
        ops = kernels.current()
        resid = torch.empty((batch.num_tokens, self.spec.hidden), dtype=torch.float32, device=self.device)
        ops.embed(self.embed, batch.token_ids, resid)
        if self.input_position is not None:
            self.input_position.add_to_stream(resid, batch)
        if observer is not None:
            observer(0, resid.clone())
        delta = None
        n = len(self.run_order)
        for i, e in enumerate(self.run_order):
            block = self.blocks[e.block]
            # the block that runs next may offer buffers that let this block's last product prepare
            # its first norm
            tgt = None
            if i + 1 < n and getattr(block, "passes_emit", False):
                nxt = self.blocks[self.run_order[i + 1].block]
                if hasattr(nxt, "entry_target"):
                    tgt = nxt.entry_target(resid)
            if tgt is not None:
                delta = block.forward(resid, delta, batch, caches[i], emit=tgt)
            else:
                delta = block.forward(resid, delta, batch, caches[i])
            if observer is not None:
                # the block's last addend may not be in the stream yet
                observer(i + 1, resid + delta.float() if isinstance(delta, torch.Tensor) else resid.clone())
        return resid, delta

    def forward(self, batch, caches: Sequence[Optional[LayerCache]], observer=None) -> torch.Tensor:
        """Logits [len(batch.logit_rows), vocab] in float32 for the step's tokens.

        The head runs on the wanted rows only (the reference computes all rows of
        a prompt and keeps the last, crates/cuda/src/engine.rs:5685-5720)."""
        resid, delta = self.forward_layers(batch, caches, observer)
        if delta is not None and not isinstance(delta, torch.Tensor):
            delta = None               # a filled norm target: the sum is already in the stream
        xn = self.final_norm.add_norm(resid, delta, rows=batch.logit_rows)
        logits = torch.empty((batch.num_logit_rows, self.spec.vocab_size), dtype=torch.float32,
                             device=self.device)
        kernels.current().linear(xn, self.head, logits)
        return logits
