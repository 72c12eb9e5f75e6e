"""What a mixer asks of the cache, and what a layer is handed at run time."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

import torch


@dataclass(frozen=True)
class PagedNeed:
    """Memory per token, in pages: the mixer names the tensors it keeps and the shape of one block of
    each. ``tensors`` is a tuple of (name, shape of one block, dtype or None for the model's dtype), a -1
    in a shape standing for the engine's block size; the
    engine allocates ``[blocks, *shape]`` for each and hands them over in ``LayerCache.tensors`` by name;
    token slot s of the step (``batch.slots[group]``) is slot ``s % block_size`` of block ``s // block_size``,
    wherever in its block's shape the mixer puts it. ``window`` W > 0: only the last W tokens are read, the
    blocks behind them go back to the pool."""
    tensors: Tuple[Tuple[str, Tuple[int, ...], Optional[torch.dtype]], ...]
    window: int = 0

    def block_tensors(self, block_size: int):
        return tuple((name, tuple(block_size if n == -1 else n for n in shape), dtype)
                     for name, shape, dtype in self.tensors)


@dataclass(frozen=True)
class KVNeed:
    """Keys and values of every token (``window`` 0) or of the last ``window`` tokens, as the attention
    kernels read them: tensors "k" and "v", a block of each ``[kv_heads, block_size // 16, 16 * head_dim]``,
    tiles of 16 slots in matrix-core operand order (:mod:`reinfer_amd.cache.layout`)."""
    num_kv_heads: int
    head_dim: int
    window: int = 0

    def block_tensors(self, block_size: int):
        from ..cache.layout import cache_shape
        shape = cache_shape(1, self.num_kv_heads, block_size, self.head_dim)[1:]
        return (("k", shape, None), ("v", shape, None))


@dataclass(frozen=True)
class StateNeed:
    """Per-request state of fixed size: one ``shape`` tensor per live request."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class LayerCache:
    """The cache of one run-order entry, as its mixer sees it.

    Paged memory: ``tensors[name]`` is ``[blocks, *shape of one block]`` as the mixer's need named it;
    for keys and values (:class:`KVNeed`) ``k``/``v`` are the same tensors,
    ``[blocks, kv_heads, block_size // 16, 16 * head_dim]``, tiles of 16 slots in the order of
    :mod:`reinfer_amd.cache.layout`; ``group`` picks the step's block tables and slots, ``writes`` is
    False for an entry that reads another entry's cache. For state: ``state`` is
    ``[max_seqs, *shape]``, indexed by the step's ``state_slots``.
    """
    k: Optional[torch.Tensor] = None
    v: Optional[torch.Tensor] = None
    group: int = 0
    writes: bool = True
    state: Optional[torch.Tensor] = None
    tensors: Optional[dict] = None      # every paged tensor by the name its mixer gave it ("k" and "v" among them)


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
    may be given one (``emit=``); it returns it if it filled it.

    ``finished``: with more rows than a product behind the norm could scale (they are the library's), the
    part is asked for the whole norm instead, ``x`` = bfloat16(norm(new stream) * norm.weight), and there are
    no sums; it returns the target only if its product could do that."""
    norm: object
    x: torch.Tensor
    ss: Optional[torch.Tensor]
    finished: bool = False

    @property
    def emit(self):
        return self.norm.weight, self.x, self.ss

    @property
    def finish(self):
        return self.norm.weight, self.x, self.norm.eps


def split_input(x):
    """(tensor, row sums or None) of a part's input, plain or :class:`RowScaled`."""
    if isinstance(x, RowScaled):
        return x.x, x.row_sums
    return x, None
