"""How the prompt attention's query tiles are listed for its kernel: host arithmetic, no GPU."""
import random

from reinfer_amd.kernels.ops import HipKernels

ROOM = 32


def plan(portions, room=ROOM, halves=True, tile=64):
    """``portions``: (tokens, tokens already cached) of each request of a step."""
    ops = HipKernels.__new__(HipKernels)         # the choice needs no loaded library
    tiles, row = [], 0
    for i, (n, start) in enumerate(portions):
        for q0 in range(0, n, tile):
            tiles.append((i, row + q0, min(tile, n - q0), start + q0))
        row += n
    return tiles, ops._prefill_items(tiles, room, halves)


def covered(tiles, items, merge, n_slots):
    """Every (tile, head half, key) is in exactly one item; parts of a tile own consecutive slots."""
    ROUND = HipKernels.PREFILL_ROUND
    seen = {}
    for cost, (i, row, nq, pos), lo, hi, slot in items:
        assert cost > 0
        q, bits = nq & 0xffff, nq >> 16
        keys = pos + q
        lo, hi = (0, keys) if slot < 0 else (lo, min(hi, keys))
        assert lo % ROUND == 0 and lo < hi, "a part starts at a round and holds a key"
        for half in ((1, 2) if bits == 0 else (bits,)):
            seen.setdefault((i, row, q, pos, half), []).append((lo, hi, slot))
    assert set(k[:4] for k in seen) == set(tiles)
    slots_used = []
    for (i, row, q, pos, half), spans in seen.items():
        spans.sort()
        assert spans[0][0] == 0 and spans[-1][1] == pos + q
        for a, b in zip(spans, spans[1:]):
            assert a[1] == b[0], "parts neither overlap nor leave a gap"
        if len(spans) > 1:
            assert [s[2] for s in spans] == list(range(spans[0][2], spans[0][2] + len(spans)))
            if half == 1:
                slots_used.append((row, q, spans[0][2], len(spans)))
        else:
            assert spans[0][2] == -1
    listed = sorted(tuple(merge[4 * k:4 * k + 4]) for k in range(len(merge) // 4))
    assert listed == sorted(slots_used)
    assert n_slots == sum(m[3] for m in listed)
    assert sorted(s for m in listed for s in range(m[2], m[2] + m[3])) == list(range(n_slots))


def test_a_whole_prompt_that_fills_the_chip_lists_its_heaviest_tiles_twice_by_heads():
    tiles, (items, merge, n_slots) = plan([(2048, 0)])
    covered(tiles, items, merge, n_slots)
    assert n_slots == 0 and len(items) == len(tiles) + ROOM // 4
    halved = {it[1][3] for it in items if it[1][2] >> 16}
    assert halved == {pos for (_, _, _, pos) in sorted(tiles, key=lambda t: -t[3])[:ROOM // 4]}


def test_without_halves_a_whole_prompt_is_listed_as_it_is():
    tiles, (items, merge, n_slots) = plan([(2048, 0)], halves=False)
    assert [it[1] for it in items] == tiles and not merge and n_slots == 0


def test_a_portion_deep_in_a_long_prompt_is_cut_by_keys_to_fill_the_chip():
    for portion in ((512, 3584), (256, 7936), (64, 4000), (256, 1792)):
        tiles, (items, merge, n_slots) = plan([portion])
        covered(tiles, items, merge, n_slots)
        assert n_slots > 0 and len(items) <= ROOM
        assert all(it[4] >= 0 for it in items), "every tile is heavy: each is cut"
        heaviest = max(it[0] for it in items)
        whole = max(-(-(pos + q) // 64) for (_, _, q, pos) in tiles)
        assert heaviest <= whole / 3
        per_tile = {}
        for it in items:
            per_tile[it[1]] = per_tile.get(it[1], 0) + 1
        assert max(per_tile.values()) <= HipKernels.PREFILL_MAX_PARTS


def test_a_full_chip_of_heavy_tiles_is_left_alone():
    # 32 tiles of 33 to 64 rounds: no room for parts, and a half that queues behind a tile of 33 rounds ends last
    tiles, (items, merge, n_slots) = plan([(2048, 2048)])
    assert [it[1] for it in items] == tiles and n_slots == 0
    # more tiles than the chip holds
    tiles, (items, merge, n_slots) = plan([(3072, 0)])
    assert [it[1] for it in items] == tiles and n_slots == 0


def test_short_parts_are_not_made():
    tiles, (items, merge, n_slots) = plan([(64, 300)])       # 6 rounds: parts of 4 at least
    assert n_slots == 0
    tiles, (items, merge, n_slots) = plan([(64, 500)])       # 9 rounds: two halves by heads cost less than two parts and their sum
    assert n_slots == 0 and len(items) == 2
    tiles, (items, merge, n_slots) = plan([(64, 700)])       # 12 rounds: three parts of 4
    assert n_slots == 3
    covered(tiles, items, merge, n_slots)


def test_random_steps_are_covered_once():
    rng = random.Random(5)
    for _ in range(300):
        portions = [(rng.randint(5, 700), rng.choice((0, 0, rng.randint(0, 9000)))) for _ in range(rng.randint(1, 6))]
        room = rng.choice((0, 4, 16, 32, 64))
        tiles, (items, merge, n_slots) = plan(portions, room=room, halves=rng.random() < 0.7,
                                              tile=rng.choice((16, 32, 64)))
        covered(tiles, items, merge, n_slots)


def test_span_starts_the_heaviest_first():
    span = HipKernels._span
    assert span([3, 9, 4], 4) == 9
    assert span([5, 5, 5, 5], 2) == 10
    assert span([8, 1, 1, 1, 1, 6], 2) == 9          # 8 | 6 1 1 1: the fourth 1 goes behind the 8
