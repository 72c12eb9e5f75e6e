"""What a mixer asks of the cache, and what a layer is handed at run time."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

import torch


@dataclass(frozen=True)
class KVNeed:
    """Keys and values of every token (``window`` 0) or of the last ``window`` tokens."""
    num_kv_heads: int
    head_dim: int
    window: int = 0


@dataclass(frozen=True)
class StateNeed:
    """Per-request state of fixed size: one ``shape`` tensor per live request."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class LayerCache:
    """The cache of one run-order entry, as its mixer sees it.

    For keys and values: ``k``/``v`` are ``[blocks, kv_heads, block_size // 16, 16 * head_dim]``,
    tiles of 16 slots in the order of :mod:`reinfer_amd.cache.layout`;
    ``group`` picks the step's block tables and slots, ``writes`` is False for an
    entry that reads another entry's cache. For state: ``state`` is
    ``[max_seqs, *shape]``, indexed by the step's ``state_slots``.
    """
    k: Optional[torch.Tensor] = None
    v: Optional[torch.Tensor] = None
    group: int = 0
    writes: bool = True
    state: Optional[torch.Tensor] = None


@dataclass
class RowScaled:
    """Rows whose RMSNorm is half done: ``x`` = bfloat16(stream * norm weight) [T, width]; the
    row factor rsqrt(sum_p ss[p, t] / width + eps) is applied by the product that takes them
    (y = rstd * ((x .* w) . W^T): the norm costs no kernel of its own). A part that declares
    ``takes_row_scaled = True`` may be handed this instead of a tensor."""
    x: torch.Tensor
    ss: torch.Tensor            # float32 [parts, T]
    eps: float
    width: int

    @property
    def row_sums(self):
        return self.ss, self.eps, self.width


@dataclass
class NormTarget:
    """Buffers that a part's last product fills for the norm that follows it, when it adds its
    result into the stream itself: ``x`` = bfloat16(new stream * norm.weight), ``ss`` = partial
    sums of squares of the new stream's rows. A part that declares ``emits_for_norm = True``
    may be given one (``emit=``); it returns it if it filled it."""
    norm: object
    x: torch.Tensor
    ss: torch.Tensor

    @property
    def emit(self):
        return self.norm.weight, self.x, self.ss


def split_input(x):
    """(tensor, row sums or None) of a part's input, plain or :class:`RowScaled`."""
    if isinstance(x, RowScaled):
        return x.x, x.row_sums
    return x, None
