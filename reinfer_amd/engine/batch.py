"""One step's work as the kernels see it: a ragged batch of token runs.

Every request in the step brings its next tokens (a portion of its prompt, or a
single decoded token); token j of a request that already holds ``start`` tokens
sits at position ``start + j`` and reads keys [0, start + j] of that request
through its block table. All index arrays are int32, packed into one host
buffer and sent to the device in one copy.

The reference has two separate calls instead, a whole prompt from position 0
(crates/cuda/src/engine.rs:5218) or one token per request (engine.rs:5853,
``BatchReq {token, pos, kv}`` at :1684-1715), and never both in a step.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Sequence

import torch

from .._hostlib import host as _host

# A request's part in a step, ``StepEntry(rid, tokens, want=[])``: its next tokens and the
# indices into them where logits are wanted. Kept by the host runtime so that checking,
# block growth and packing read it without a call back into Python.
StepEntry = _host.StepEntry


@dataclass
class StepBatch:
    num_tokens: int
    num_seqs: int
    num_logit_rows: int
    # device tensors (int32)
    token_ids: torch.Tensor         # [T]
    positions: torch.Tensor         # [T]
    seq_of_token: torch.Tensor      # [T]   index of the token's request in this step
    cu_tokens: torch.Tensor         # [n+1] first token of each request in the step
    start_pos: torch.Tensor         # [n]   tokens the request held before the step
    ctx_lens: torch.Tensor          # [n]   tokens it holds after the step
    state_slots: torch.Tensor       # [n]   per-request state slot
    fresh: torch.Tensor             # [n]   1 if this is the request's first step
    logit_rows: Optional[torch.Tensor]   # [n_out] token rows whose logits are wanted
    no_slots: torch.Tensor          # [T]   all -1: "store nothing"
    block_tables: List[torch.Tensor]     # per cache group [n, width]
    slots: List[torch.Tensor]            # per cache group [T] flat cache slot of each token
    # host copies, for choosing kernels and grids without a device read
    q_lens: List[int] = field(default_factory=list)
    starts: List[int] = field(default_factory=list)
    max_q_len: int = 0
    max_ctx_len: int = 0
    extra: dict = field(default_factory=dict)     # kernel-specific device arrays, made on demand


def build_step_batch(entries: Sequence[StepEntry], manager, device: torch.device,
                     pin: bool = False) -> StepBatch:
    """Pack index arrays for ``entries``; the manager already holds their blocks.
    The host runtime fills the buffer (CacheManager.fill_step)."""
    entries = list(entries)
    n = len(entries)
    n_groups = len(manager.groups)
    q_lens, starts, widths, n_out = manager.step_shape(entries)
    T = sum(q_lens)

    # layout of the packed buffer
    sizes = [T, T, T, n + 1, n, n, n, n, max(n_out, 1), T]
    sizes += [n * w for w in widths] + [T] * n_groups
    offs = [0]
    for s in sizes:
        offs.append(offs[-1] + s)
    host = torch.zeros(offs[-1], dtype=torch.int32, pin_memory=pin)
    manager.fill_step(entries, host.numpy(), offs[:-1], widths)

    dev = host.to(device, non_blocking=pin)

    def view(k: int, shape=None) -> torch.Tensor:
        v = dev[offs[k]:offs[k + 1]]
        return v if shape is None else v.view(shape)

    return StepBatch(
        num_tokens=T, num_seqs=n, num_logit_rows=n_out,
        token_ids=view(0), positions=view(1), seq_of_token=view(2), cu_tokens=view(3),
        start_pos=view(4), ctx_lens=view(5), state_slots=view(6), fresh=view(7),
        logit_rows=view(8)[:n_out] if n_out else None, no_slots=view(9),
        block_tables=[view(10 + g, (n, widths[g])) for g in range(n_groups)],
        slots=[view(10 + n_groups + g) for g in range(n_groups)],
        q_lens=list(q_lens), starts=list(starts), max_q_len=max(q_lens),
        max_ctx_len=max(s + q for s, q in zip(starts, q_lens)))
