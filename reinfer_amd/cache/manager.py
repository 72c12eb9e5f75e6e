"""Paged cache bookkeeping (host only): block pools, block tables, state slots.

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


class OutOfBlocks(RuntimeError):
    """A pool cannot give the blocks asked for (crates/memory/src/pool.rs OutOfPages{need, free})."""

    def __init__(self, group: int, need: int, free: int):
        super().__init__(f"cache group {group}: need {need} blocks, {free} free")
        self.group, self.need, self.free = group, need, free


class OutOfSlots(RuntimeError):
    pass


class BlockPool:
    """Fixed set of block ids with a LIFO free list; every misuse is an error."""

    def __init__(self, num_blocks: int):
        if num_blocks <= 0:
            raise ValueError("a pool needs at least one block")
        self.num_blocks = num_blocks
        self._free: List[int] = list(range(num_blocks - 1, -1, -1))   # pop() gives 0 first
        self._held = [False] * num_blocks
        self.allocs = 0
        self.frees = 0

    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_held(self) -> int:
        return self.num_blocks - len(self._free)

    def take(self) -> int:
        if not self._free:
            raise OutOfBlocks(-1, 1, 0)
        b = self._free.pop()
        assert not self._held[b], f"block {b} handed out twice"
        self._held[b] = True
        self.allocs += 1
        return b

    def give_back(self, b: int) -> None:
        if not 0 <= b < self.num_blocks:
            raise ValueError(f"block {b} is not of this pool")
        if not self._held[b]:
            raise RuntimeError(f"block {b} freed twice")
        self._held[b] = False
        self._free.append(b)
        self.frees += 1

    def check(self) -> None:
        assert len(set(self._free)) == len(self._free), "a block is on the free list twice"
        assert all(not self._held[b] for b in self._free), "a free block is marked held"
        assert sum(self._held) + len(self._free) == self.num_blocks, "a block is lost"
        assert self.allocs - self.frees == self.num_held


class SlotPool:
    """Ids for per-request state of fixed size."""

    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self._free = list(range(num_slots - 1, -1, -1))
        self._held = [False] * num_slots

    @property
    def num_free(self) -> int:
        return len(self._free)

    def take(self) -> int:
        if not self._free:
            raise OutOfSlots(f"all {self.num_slots} request slots are in use")
        s = self._free.pop()
        self._held[s] = True
        return s

    def give_back(self, s: int) -> None:
        if not self._held[s]:
            raise RuntimeError(f"slot {s} freed twice")
        self._held[s] = False
        self._free.append(s)


@dataclass(frozen=True)
class CacheGroupSpec:
    """Layers (run-order entries) that share block tables. ``window`` 0: all keys."""
    window: int
    entries: Tuple[int, ...]


@dataclass
class RequestCache:
    slot: int
    num_tokens: int = 0                     # tokens whose keys are stored
    tables: List[List[int]] = field(default_factory=list)   # per group; -1 = given back
    first_live: List[int] = field(default_factory=list)     # per group: first block still held
    fresh: bool = True                      # no step has run for it yet


class CacheManager:
    def __init__(self, groups: Sequence[CacheGroupSpec], block_size: int,
                 num_blocks: Sequence[int], max_seqs: int):
        if block_size <= 0:
            raise ValueError("block_size must be positive")
        if len(num_blocks) != len(groups):
            raise ValueError("one block count per cache group")
        self.groups = list(groups)
        self.block_size = block_size
        self.pools = [BlockPool(n) for n in num_blocks]
        self.slots = SlotPool(max_seqs)
        self.requests: Dict[Hashable, RequestCache] = {}

    # ------------------------------------------------------------- requests
    def add(self, rid: Hashable) -> RequestCache:
        if rid in self.requests:
            raise KeyError(f"request {rid!r} is already live")
        rc = RequestCache(slot=self.slots.take(), tables=[[] for _ in self.groups],
                          first_live=[0 for _ in self.groups])
        self.requests[rid] = rc
        return rc

    def get(self, rid: Hashable) -> RequestCache:
        return self.requests[rid]

    def __contains__(self, rid: Hashable) -> bool:
        return rid in self.requests

    def free(self, rid: Hashable) -> None:
        """Give back everything a request holds, exactly once
        (crates/scheduler/src/req.rs:372-378, take_release)."""
        rc = self.requests.pop(rid, None)
        if rc is None:
            raise KeyError(f"request {rid!r} is not live (freed twice?)")
        for g, table in enumerate(rc.tables):
            for b in reversed(table):
                if b >= 0:
                    self.pools[g].give_back(b)
        self.slots.give_back(rc.slot)

    # --------------------------------------------------------------- blocks
    def _first_needed_block(self, g: int, first_query_pos: int) -> int:
        """First block a query at ``first_query_pos`` can still read in group g."""
        w = self.groups[g].window
        if w <= 0:
            return 0
        lo = first_query_pos - w + 1
        return max(0, lo) // self.block_size

    def blocks_needed(self, rid: Hashable, new_total: int) -> List[int]:
        """Blocks each group must still take so that tokens [stored, new_total) fit."""
        rc = self.requests[rid]
        need = []
        for g in range(len(self.groups)):
            have = len(rc.tables[g])
            want = -(-new_total // self.block_size)
            # blocks wholly below the window of the first new query are never taken
            first = max(have, self._first_needed_block(g, rc.num_tokens))
            need.append(max(0, want - first))
        return need

    def can_grow(self, growth: Sequence[Tuple[Hashable, int]]) -> bool:
        total = [0] * len(self.groups)
        for rid, new_total in growth:
            for g, n in enumerate(self.blocks_needed(rid, new_total)):
                total[g] += n
        return all(total[g] <= self.pools[g].num_free for g in range(len(self.groups)))

    def grow(self, rid: Hashable, new_total: int) -> None:
        """Take the blocks for tokens up to ``new_total``; all groups or none."""
        rc = self.requests[rid]
        if new_total < rc.num_tokens:
            raise ValueError("a request's cache does not shrink")
        need = self.blocks_needed(rid, new_total)
        for g, n in enumerate(need):
            if n > self.pools[g].num_free:
                raise OutOfBlocks(g, n, self.pools[g].num_free)
        want = -(-new_total // self.block_size)
        for g in range(len(self.groups)):
            table = rc.tables[g]
            first = self._first_needed_block(g, rc.num_tokens)
            while len(table) < want:
                if len(table) < first:
                    table.append(-1)            # below the window from the start: never held
                    rc.first_live[g] = len(table)
                else:
                    table.append(self.pools[g].take())

    def commit(self, rid: Hashable, new_total: int) -> None:
        """The step has stored tokens up to ``new_total``; give back what every
        later query's window has passed."""
        rc = self.requests[rid]
        rc.num_tokens = new_total
        rc.fresh = False
        for g in range(len(self.groups)):
            first = self._first_needed_block(g, new_total)    # next query sits at new_total
            table = rc.tables[g]
            for b in range(rc.first_live[g], min(first, len(table))):
                if table[b] >= 0:
                    self.pools[g].give_back(table[b])
                    table[b] = -1
            rc.first_live[g] = max(rc.first_live[g], min(first, len(table)))

    def slot_of(self, rid: Hashable, group: int, pos: int) -> int:
        """Flat cache slot (block * block_size + offset) of position ``pos``; -1 if not held."""
        b = self.requests[rid].tables[group][pos // self.block_size]
        return -1 if b < 0 else b * self.block_size + pos % self.block_size

    # ---------------------------------------------------------------- checks
    def check(self) -> None:
        """No block lost, held twice or free while held."""
        for g, pool in enumerate(self.pools):
            pool.check()
            held = [b for rc in self.requests.values() for b in rc.tables[g] if b >= 0]
            assert len(held) == len(set(held)), f"group {g}: a block is held by two requests"
            assert len(held) == pool.num_held, f"group {g}: {pool.num_held} held, {len(held)} in tables"
            assert all(pool._held[b] for b in held)
        slots = [rc.slot for rc in self.requests.values()]
        assert len(slots) == len(set(slots)), "a state slot is held twice"
        assert len(slots) + self.slots.num_free == self.slots.num_slots

    def stats(self) -> Dict[str, object]:
        return {"block_size": self.block_size, "live_requests": len(self.requests),
                "blocks_total": [p.num_blocks for p in self.pools],
                "blocks_free": [p.num_free for p in self.pools],
                "allocs": [p.allocs for p in self.pools], "frees": [p.frees for p in self.pools]}


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
