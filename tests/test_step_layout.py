"""The native step layout: what the kernels of a step read (no GPU needed)."""
import numpy as np
import pytest

from leone_amd import ops
from leone_amd.cache.manager import CacheManager, GroupSpec
from leone_amd.engine.engine import PackedStep, StepEntry, StepError
from leone_amd.parts.base import RowTiling

PROMPT = RowTiling(ops.PREFILL_TILE_ROWS, ops.PREFILL_GROUP_TILES, ops.PREFILL_MIN_ROWS)   # the attention mixer's


def reserved(cache, entries):
    for e in entries:
        if not cache.has(e.request):
            cache.admit(e.request)
        cache.reserve(e.request, len(e.tokens))


def sections(packed):
    words = packed.host.numpy()
    return [words[packed.offsets[i]:packed.offsets[i + 1]] for i in range(len(packed.offsets) - 1)]


def test_rows_positions_tables_and_wanted_rows():
    cache = CacheManager([GroupSpec(40, 16), GroupSpec(40, 8, window=20)], max_requests=4, max_context=200)
    cache.admit("old")
    cache.reserve("old", 37)
    cache.commit("old")
    entries = [StepEntry("old", [7], [0]), StepEntry("long", list(range(100, 150)), [49, 0]),
               StepEntry("short", [1, 2, 3], [])]
    reserved(cache, entries)
    packed = PackedStep(cache, 1000, entries, tilings=[PROMPT])
    tokens, positions, row_entry, slots, want, tiles, table0, table1 = sections(packed)
    # the portion long enough for the tiled kernel runs first, the others keep their order
    assert [p[0] for p in packed.placed] == [1, 0, 2]
    assert tokens.tolist() == list(range(100, 150)) + [7] + [1, 2, 3]
    assert positions.tolist() == list(range(50)) + [37] + [0, 1, 2]
    assert row_entry.tolist() == [0] * 50 + [1] + [2] * 3
    assert slots.tolist() == [cache.slot("long"), cache.slot("old"), cache.slot("short")]
    assert want.tolist() == [50, 49, 0]                       # in the caller's order of entries and places
    assert (packed.rows, packed.tiled[0][0], packed.max_position, packed.decode_only) == (54, 50, 49, False)
    width0, width1 = cache.max_blocks(0), cache.max_blocks(1)
    for place, name in enumerate(["long", "old", "short"]):
        for table, width, group in ((table0, width0, 0), (table1, width1, 1)):
            mine = table[place * width:(place + 1) * width].tolist()
            held = cache.table(name, group)
            assert mine == held + [-1] * (width - len(held))
    listed = tiles.reshape(-1, 3).tolist()
    assert len(listed) == ops.PREFILL_GROUP_TILES
    assert listed[:2] == [[0, 0, 32], [0, 32, 18]] and all(t[0] == 0 and t[2] == 0 for t in listed[2:])


@pytest.mark.parametrize("rows", [16, 31, 32, 33, 256, 257, 300, 700, 2048])
def test_every_tile_is_listed_once_in_groups_of_one_entry(rows):
    cache = CacheManager([GroupSpec(200, 16)], max_requests=2, max_context=3000)
    other = StepEntry("b", list(range(40)), [])
    entry = StepEntry("a", [5] * rows, [rows - 1])
    reserved(cache, [other, entry])
    packed = PackedStep(cache, 100, [other, entry], tilings=[PROMPT])
    tiles = sections(packed)[5].reshape(-1, 3)
    group = ops.PREFILL_GROUP_TILES
    assert len(tiles) % group == 0
    place_of = {packed.placed[i][0]: i for i in range(2)}
    first_row = {i: packed.placed[place_of[i]][2] for i in range(2)}
    covered = {0: [], 1: []}
    for g in range(0, len(tiles), group):
        members = tiles[g:g + group]
        assert len(set(members[:, 0].tolist())) == 1           # one entry a group
        given = [i for i in range(2) if place_of[i] == members[0, 0]][0]
        used = members[members[:, 2] > 0]
        for _, start, count in used.tolist():
            assert 0 < count <= ops.PREFILL_TILE_ROWS
            covered[given] += list(range(start - first_row[given], start - first_row[given] + count))
    assert sorted(covered[1]) == list(range(rows)) and sorted(covered[0]) == list(range(40))


def test_decode_layout_wants_every_row():
    cache = CacheManager([GroupSpec(8, 16)], max_requests=3, max_context=64)
    entries = [StepEntry(i, [i + 1], [0] if i else []) for i in range(3)]
    reserved(cache, entries)
    packed = PackedStep(cache, 10, entries, all_rows_wanted=True, tilings=[PROMPT])
    tokens, positions, row_entry, slots, want, tiles = sections(packed)[:6]
    assert tokens.tolist() == [1, 2, 3] and want.tolist() == [0, 1, 2] and tiles.size == 0 and packed.decode_only


@pytest.mark.parametrize("entries, message", [
    ([], "at least one"), ([StepEntry("a", [1]), StepEntry("a", [2])], "twice"), ([StepEntry("a", [])], "no tokens"),
    ([StepEntry("a", [10])], "vocabulary"), ([StepEntry("a", [-1])], "vocabulary"),
    ([StepEntry("a", [1, 2], [2])], "wanted place"), ([StepEntry("nobody", [1])], "not admitted"),
])
def test_malformed_steps_are_refused(entries, message):
    cache = CacheManager([GroupSpec(8, 16)], max_requests=3, max_context=64)
    cache.admit("a")
    with pytest.raises(StepError, match=message):
        PackedStep(cache, 10, entries)


def test_two_tilings_each_find_their_portions_at_the_front():
    """Parts with kernels of different shapes each declare a tiling; the entries that more tilings cut come
    first, so the rows of a tiling's portions are the step's first rows whatever its threshold; a model
    without any gets no tile list at all."""
    cache = CacheManager([GroupSpec(100, 16)], max_requests=6, max_context=400)
    entries = [StepEntry("one", [1], [0]), StepEntry("mid", [2] * 10, []), StepEntry("long", [3] * 70, [69]),
               StepEntry("two", [4, 4], []), StepEntry("mid2", [5] * 24, [0])]
    reserved(cache, entries)
    coarse, fine = RowTiling(32, 4, 16), RowTiling(8, 2, 5)
    packed = PackedStep(cache, 10, entries, tilings=[coarse, fine])
    assert [p[0] for p in packed.placed] == [2, 4, 1, 0, 3]      # cut by both, by the fine one only, by none
    tokens, positions, row_entry, slots, want, tiles_coarse, tiles_fine, table = sections(packed)
    assert packed.tiled == [(94, 8), (104, 16)]                  # (rows, tile places) of each
    assert tiles_coarse.reshape(-1, 3).tolist() == [[0, 0, 32], [0, 32, 32], [0, 64, 6], [0, 0, 0],
                                                    [1, 70, 24], [1, 70, 0], [1, 70, 0], [1, 70, 0]]
    listed = tiles_fine.reshape(-1, 3).tolist()
    assert listed[:9] == [[0, 8 * i, 8] for i in range(8)] + [[0, 64, 6]] and listed[9] == [0, 0, 0]
    assert listed[10:14] == [[1, 70, 8], [1, 78, 8], [1, 86, 8], [1, 70, 0]]
    assert listed[14:] == [[2, 94, 8], [2, 102, 2]]
    assert want.tolist() == [104, 69, 70]
    none = PackedStep(cache, 10, entries)
    assert none.tiled == [] and len(sections(none)) == 6 and [p[0] for p in none.placed] == [0, 1, 2, 3, 4]
