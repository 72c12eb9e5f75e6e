"""The cache manager: no block lost, held twice or freed twice, under random orders
of requests; window groups give blocks back as the window passes; slots."""
import random

import pytest

from reinfer_amd.cache import (BlockPool, CacheGroupSpec, CacheManager, OutOfBlocks, OutOfSlots, SlotPool,
                               plan_groups)


def test_pool_conservation_and_lifo():
    """crates/memory/src/pool.rs:180-235: in_use + free == total, LIFO reuse, double free."""
    p = BlockPool(4)
    a, b = p.take(), p.take()
    assert (a, b) == (0, 1) and p.num_free == 2 and p.num_held == 2
    p.give_back(a)
    assert p.take() == a                       # last freed, first used again
    p.give_back(b)
    with pytest.raises(RuntimeError, match="freed twice"):
        p.give_back(b)
    with pytest.raises(ValueError):
        p.give_back(17)
    p.check()
    c = [p.take() for _ in range(p.num_free)]
    with pytest.raises(OutOfBlocks):
        p.take()
    for x in c + [a]:
        p.give_back(x)
    assert p.num_free == 4 and p.allocs == p.frees
    p.check()


def test_slot_pool():
    s = SlotPool(2)
    a, b = s.take(), s.take()
    with pytest.raises(OutOfSlots):
        s.take()
    s.give_back(a)
    with pytest.raises(RuntimeError):
        s.give_back(a)
    assert s.take() == a


def test_plan_groups():
    groups = plan_groups([0, 8, None, 0, 8, 4])
    assert [(g.window, g.entries) for g in groups] == [(0, (0, 3)), (4, (5,)), (8, (1, 4))]


def manager(num_blocks=8, windows=(0,), bs=4, max_seqs=4):
    groups = [CacheGroupSpec(window=w, entries=(i,)) for i, w in enumerate(windows)]
    return CacheManager(groups, bs, [num_blocks] * len(groups), max_seqs)


def test_lazy_growth_and_free():
    m = manager()
    m.add("a")
    assert m.blocks_needed("a", 1) == [1] and m.blocks_needed("a", 4) == [1] and m.blocks_needed("a", 5) == [2]
    m.grow("a", 5)
    m.commit("a", 5)
    assert m.get("a").tables[0] == [0, 1] and m.blocks_needed("a", 8) == [0] and m.blocks_needed("a", 9) == [1]
    assert m.slot_of("a", 0, 0) == 0 and m.slot_of("a", 0, 4) == 4 and m.slot_of("a", 0, 3) == 3
    m.add("b")
    m.grow("b", 3)
    m.commit("b", 3)
    assert m.slot_of("b", 0, 2) == 2 * 4 + 2
    m.free("a")
    with pytest.raises(KeyError):
        m.free("a")
    m.add("c")
    m.grow("c", 8)
    assert m.get("c").tables[0] == [0, 1]      # a's blocks, used again (LIFO: first block first)
    m.check()
    with pytest.raises(KeyError):
        m.add("c")


def test_out_of_blocks_takes_nothing():
    m = manager(num_blocks=3, windows=(0, 0))
    m.add("a")
    m.grow("a", 8)
    m.add("b")
    assert not m.can_grow([("b", 8)])
    assert m.can_grow([("b", 4)])
    with pytest.raises(OutOfBlocks) as e:
        m.grow("b", 8)
    assert e.value.need == 2 and e.value.free == 1
    assert m.get("b").tables == [[], []]
    m.check()


def test_window_group_gives_back_passed_blocks():
    m = manager(num_blocks=6, windows=(0, 6), bs=4)
    m.add("a")
    for total in range(1, 25):
        m.grow("a", total)
        m.commit("a", total)
        m.check()
        rc = m.get("a")
        # full group keeps everything
        assert all(b >= 0 for b in rc.tables[0])
        # window group: a query at position `total` reads keys >= total - 5
        lo = max(0, total - 6 + 1)
        for blk, b in enumerate(rc.tables[1]):
            needed = (blk + 1) * 4 > lo
            assert (b >= 0) == needed, (total, blk, rc.tables[1])
    held = sum(1 for b in m.get("a").tables[1] if b >= 0)
    assert held <= 3                           # ceil(6/4) + 1
    assert m.pools[1].frees > 0
    m.free("a")
    assert all(p.num_free == p.num_blocks for p in m.pools)


def test_long_portion_in_window_group_needs_all_its_blocks():
    m = manager(num_blocks=8, windows=(4,), bs=4)
    m.add("a")
    m.grow("a", 20)                             # the first token of the portion reads key 0
    assert sum(1 for b in m.get("a").tables[0] if b >= 0) == 5
    m.commit("a", 20)
    assert sum(1 for b in m.get("a").tables[0] if b >= 0) == 1      # keys 17..19 live in block 4


@pytest.mark.parametrize("seed", range(20))
def test_random_orders_conserve_blocks(seed):
    rng = random.Random(seed)
    m = manager(num_blocks=12, windows=(0, 5), bs=4, max_seqs=5)
    live = {}
    next_id = 0
    for _ in range(300):
        op = rng.random()
        if op < 0.25 and len(live) < 5:
            rid = f"r{next_id}"
            next_id += 1
            m.add(rid)
            live[rid] = 0
        elif op < 0.85 and live:
            rid = rng.choice(sorted(live))
            n = rng.choice([1, 1, 1, 2, 3, 7, 13])
            if m.can_grow([(rid, live[rid] + n)]):
                m.grow(rid, live[rid] + n)
                live[rid] += n
                m.commit(rid, live[rid])
            else:
                with pytest.raises(OutOfBlocks):
                    m.grow(rid, live[rid] + n)
        elif live:
            rid = rng.choice(sorted(live))
            m.free(rid)
            del live[rid]
        m.check()
    for rid in list(live):
        m.free(rid)
    m.check()
    assert all(p.num_free == p.num_blocks and p.allocs == p.frees for p in m.pools)
    assert m.slots.num_free == 5


def test_deterministic_given_the_call_sequence():
    def run():
        m = manager(num_blocks=6)
        out = []
        for rid, n in [("a", 5), ("b", 9), ("a", 8)]:
            if rid not in m:
                m.add(rid)
            m.grow(rid, n)
            m.commit(rid, n)
            out.append([list(t) for t in m.get(rid).tables])
        m.free("a")
        m.add("c")
        m.grow("c", 4)
        out.append(m.get("c").tables)
        return out
    assert run() == run()
