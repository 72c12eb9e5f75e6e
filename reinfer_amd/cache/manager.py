"""Paged cache bookkeeping (host only): block pools, block tables, state slots.
The classes are the C++ host runtime's (reinfer_amd/csrc/host/host.cpp).

Keys and values live in blocks of ``block_size`` tokens. Layers with the same
needs form a group (all earlier keys, or a window of them); every group has a
pool of its own and every request has one block table per group. Blocks are
taken lazily, when a step's tokens need them, given back when the request ends
or, in a window group, when the window has passed them, and used again, last
freed first (the reference's ``PagePool`` is LIFO the same way,
crates/memory/src/pool.rs:61-155). Beside the pools there are slots for
per-request state of fixed size (one id per live request).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple


from .._hostlib import OutOfBlocks, OutOfSlots, host

BlockPool = host.BlockPool            # fixed set of block ids with a LIFO free list; every misuse is an error
SlotPool = host.SlotPool              # ids for per-request state of fixed size
RequestCache = host.RequestCache      # slot, num_tokens, tables (per group; -1 = given back), first_live, fresh
CacheManager = host.CacheManager      # (groups, block_size, num_blocks per group, max_seqs)


@dataclass(frozen=True)
class CacheGroupSpec:
    """Layers (run-order entries) that share block tables. ``window`` 0: all keys."""
    window: int
    entries: Tuple[int, ...]


def plan_groups(windows: Sequence[Optional[int]]) -> List[CacheGroupSpec]:
    """Group run-order entries by what they keep.

    ``windows[i]`` is None for an entry without keys of its own (it reads
    another entry's cache, or keeps fixed-size state), 0 for all keys, W > 0 for
    a window. Entries with equal needs share a group.
    """
    by: Dict[int, List[int]] = {}
    for i, w in enumerate(windows):
        if w is None:
            continue
        by.setdefault(int(w), []).append(i)
    return [CacheGroupSpec(window=w, entries=tuple(es)) for w, es in sorted(by.items())]
