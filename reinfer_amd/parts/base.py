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
