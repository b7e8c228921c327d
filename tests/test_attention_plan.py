"""The host-side work list of the attention kernels: every (token, head) pair of a step is some
item's or some workgroup tile's, with exactly the keys it may see; split key ranges tile their
range without gaps; captured steps get arrays whose shape does not depend on the contexts."""
import random

import numpy as np
import pytest

from llmserver_amd.parts.attention import (DEFAULT_TUNING, KEY_ALIGN, MAX_SPLITS, MIN_TILES_FOR_WORKGROUPS, build_attention_plan, fixed_split_count,
                                           group_tiling)


def covered_tokens(plan, row_len, row_ctx, group_size, window):
    """(row, token) -> list of (k_begin, k_end) it is computed against, over items and workgroup tiles."""
    _, tokens_per_tile, _ = group_tiling(group_size)
    seen = {}
    for (row, q0, k_begin, k_end) in plan.items.tolist():
        for token in range(q0, min(q0 + tokens_per_tile, row_len[row])):
            seen.setdefault((row, token), []).append((k_begin, k_end))
    span = plan.tiles_per_workgroup * tokens_per_tile
    for (row, q0, k_begin, k_end) in plan.tiles.tolist():
        assert plan.tiles_per_workgroup in (4, 8)
        for token in range(q0, min(q0 + span, row_len[row])):
            seen.setdefault((row, token), []).append((k_begin, k_end))
    return seen


def slots_of_tiles(plan, row_len, group_size):
    """{(row, first token of a tile): slots its key ranges write}, over the entries of ``tiles`` that have slots."""
    _, tokens_per_tile, _ = group_tiling(group_size)
    written = {}
    if plan.tile_slots is None:
        return written
    assert plan.tile_slots.shape == (len(plan.tiles), 2) and plan.tile_slots.dtype == np.int32
    for (row, q0, _, _), (first, stride) in zip(plan.tiles.tolist(), plan.tile_slots.tolist()):
        if first < 0:
            continue
        tiles_here = -(-min(plan.tiles_per_workgroup * tokens_per_tile, row_len[row] - q0) // tokens_per_tile)
        for j in range(tiles_here):
            written.setdefault((row, q0 + j * tokens_per_tile), []).append(first + j * stride)
    return written


@pytest.mark.parametrize("seed", range(40))
def test_every_token_meets_its_keys_exactly_once(seed):
    rng = random.Random(seed)
    group_size = rng.choice([1, 2, 4, 5, 8, 16, 20])
    n_kv = rng.choice([1, 2, 8])
    window = rng.choice([None, None, 40, 700])
    rows = rng.randint(1, 9)
    row_len = [rng.choice([1, 1, 1, 2, 7, 33, 200, 900]) for _ in range(rows)]
    row_ctx = [n + rng.choice([0, 0, 5, 64, 1000, 5000]) for n in row_len]
    most = rng.choice([0, 4, 8])
    key_ranges = rng.choice([1, 128, 128, 5])
    plan = build_attention_plan(row_len, row_ctx, group_size, n_kv, window, workgroup_tiles=most, tile_key_ranges=key_ranges,
                                tile_halves=rng.choice([1, 2]))
    _, tokens_per_tile, _ = group_tiling(group_size)
    seen = covered_tokens(plan, row_len, row_ctx, group_size, window)
    for row in range(rows):
        first_pos = row_ctx[row] - row_len[row]
        for token in range(row_len[row]):
            ranges = sorted(seen[(row, token)])
            # the ranges follow one another without a gap or an overlap ...
            for (a0, a1), (b0, b1) in zip(ranges, ranges[1:]):
                assert a1 == b0 or (b0 == b1), (ranges, row, token)
            lo, hi = ranges[0][0], max(r[1] for r in ranges)
            # ... and hold every key the token may see: up to itself, from the window's edge (a tile's range is that of
            # all its tokens, the kernel masks the rest)
            position = first_pos + token
            assert hi >= position + 1
            assert lo <= (0 if window is None else max(0, position - window + 1))
            if window is None:
                assert lo == 0
    # slots: one per split item and per tile and key range of a workgroup's tiles, consecutive within a merge, none
    # written twice, none left over
    slots = plan.item_slot.tolist()
    of_tiles = slots_of_tiles(plan, row_len, group_size)
    used = sorted([s for s in slots if s >= 0] + [s for written in of_tiles.values() for s in written])
    assert used == list(range(plan.n_slots))
    for (row, q0, first_slot, count) in plan.merges.tolist():
        assert 1 < count <= MAX_SPLITS or (row, q0) not in of_tiles
        if (row, q0) in of_tiles:
            assert sorted(of_tiles.pop((row, q0))) == list(range(first_slot, first_slot + count)) and count <= key_ranges
            continue
        members = [i for i, s in enumerate(slots) if first_slot <= s < first_slot + count]
        assert len(members) == count and count <= MAX_SPLITS
        assert all(plan.items[i][0] == row and plan.items[i][1] == q0 for i in members)
        begins = [int(plan.items[i][2]) for i in members]
        assert all(b % KEY_ALIGN == 0 for b in begins[1:])
    assert not of_tiles                                                       # every tile with slots has its merge
    assert sum(c for *_, c in plan.merges.tolist()) == plan.n_slots
    # key ranges of a workgroup's tiles begin at multiples of KEY_ALIGN (but the first) and none is empty
    if plan.tile_slots is not None:
        for (_, _, k_begin, k_end), (first, stride) in zip(plan.tiles.tolist(), plan.tile_slots.tolist()):
            assert k_begin < k_end and (first < 0 or stride > 1)
        groups = {}
        for (row, q0, k_begin, k_end), (first, stride) in zip(plan.tiles.tolist(), plan.tile_slots.tolist()):
            groups.setdefault((row, q0), []).append((k_begin, k_end, first, stride))
        for ranges in groups.values():
            ranges.sort()
            assert all(b[0] % KEY_ALIGN == 0 for b in ranges[1:]) and all(a[1] == b[0] for a, b in zip(ranges, ranges[1:]))
            assert len(ranges) == 1 or ([r[2] for r in ranges] == list(range(ranges[0][2], ranges[0][2] + len(ranges)))
                                        and all(r[3] == len(ranges) for r in ranges))
    # rows with many tiles go to the workgroup kernel when it is offered, and only those; rows of few tiles too if the
    # kernel can cut their keys into ranges
    tiles_per_row = [-(-n // tokens_per_tile) for n in row_len]
    rows_in_tiles = {int(r) for r in plan.tiles[:, 0]} if len(plan.tiles) else set()
    enough = MIN_TILES_FOR_WORKGROUPS if key_ranges == 1 else DEFAULT_TUNING.min_tiles_with_ranges
    expected = {r for r in range(rows) if most and tiles_per_row[r] >= enough}
    if sum(tiles_per_row[r] for r in expected) < MIN_TILES_FOR_WORKGROUPS:      # too few tiles for a launch of their own
        expected = set()
    assert rows_in_tiles == expected
    keys_of_tiles = [int(k_end - k_begin) for _, _, k_begin, k_end in plan.tiles.tolist()]
    assert keys_of_tiles == sorted(keys_of_tiles, reverse=True)              # the longest start first


def test_captured_steps_get_arrays_of_one_shape():
    group_size, n_kv = 4, 8
    rows = 5
    fixed = fixed_split_count(rows, group_size, n_kv, 4096)
    shapes = set()
    for contexts in ([1] * rows, [4096] * rows, [1, 17, 300, 2049, 4000], [33] * rows):
        plan = build_attention_plan([1] * rows, contexts, group_size, n_kv, None, fixed_splits=fixed)
        shapes.add((plan.items.shape, plan.item_slot.shape, plan.merges.shape, plan.n_slots, plan.tiles.shape))
        for (row, q0, k_begin, k_end) in plan.items.tolist():
            assert 0 <= k_begin <= k_end <= contexts[row]
        # exactly one item of a row ends at its context and is not empty: the one that takes the new token
        for row in range(rows):
            ending = [(b, e) for (r, _, b, e) in plan.items.tolist() if r == row and e == contexts[row] and b < e]
            assert len(ending) == 1
    assert len(shapes) == 1
    assert fixed_split_count(64, group_size, n_kv, 4096) < fixed_split_count(1, group_size, n_kv, 4096)


@pytest.mark.parametrize("seed", range(20))
def test_plan_of_single_tokens_made_at_once_equals_the_plan_made_row_by_row(seed):
    rng = random.Random(seed)
    rows = rng.randint(1, 70)
    contexts = [rng.choice((1, 2, 31, 32, 33, 64, 100, 1000, 4095, 4096, 4097, rng.randint(1, 9000))) for _ in range(rows)]
    window = rng.choice((None, None, 1, 40, 700))
    splits = rng.choice((1, 2, 3, 8, 16, 128))
    group_size, n_kv = rng.choice((1, 4, 20)), rng.choice((1, 8))
    fast = build_attention_plan([1] * rows, contexts, group_size, n_kv, window, fixed_splits=splits)
    slow = build_attention_plan([1] * rows, contexts, group_size, n_kv, window, fixed_splits=splits, single_token_shortcut=False)
    for name in ("items", "item_slot", "merges", "tiles"):
        a, b = getattr(fast, name), getattr(slow, name)
        assert a.dtype == b.dtype and a.shape == b.shape and (a == b).all(), name
    assert fast.n_slots == slow.n_slots and fast.tiles_per_workgroup == slow.tiles_per_workgroup


@pytest.mark.parametrize("seed", range(10))
def test_plan_whose_key_ranges_are_merged_in_the_workgroup(seed):
    """Four items a row, in the row's order, without slots or merges; the ranges follow one another from the first key
    the token may see to itself, at multiples of KEY_ALIGN; empty ranges lie at the end."""
    rng = random.Random(seed)
    rows = rng.randint(1, 70)
    contexts = [rng.choice((1, 2, 31, 32, 33, 64, 100, 300, 511, 512, 513, 1024, rng.randint(1, 2000))) for _ in range(rows)]
    window = rng.choice((None, None, 1, 40, 700))
    per_tile = rng.choice((4, 4, 2))               # two ranges a tile: two tiles to a workgroup, rows in pairs
    if per_tile == 2 and rows % 2:
        with pytest.raises(ValueError):
            build_attention_plan([1] * rows, contexts, 4, 8, window, merge_in_workgroup=2)
        rows, contexts = rows + 1, contexts + [77]
    plan = build_attention_plan([1] * rows, contexts, rng.choice((1, 4, 20)), rng.choice((1, 8)), window, fixed_splits=rng.choice((None, 1, 16)),
                                merge_in_workgroup=per_tile)
    assert plan.merge_in_workgroup == per_tile and plan.items.shape == (per_tile * rows, 4) and plan.n_slots == 0 and plan.merges.shape == (0, 4)
    assert (plan.item_slot == -1).all() and plan.tiles.shape == (0, 4) and len(plan.items) % 4 == 0
    for row, context in enumerate(contexts):
        ranges = plan.items[per_tile * row:per_tile * row + per_tile].tolist()
        assert all(r == row and q0 == 0 for r, q0, _, _ in ranges)
        first = 0 if window is None else max(0, context - window)
        filled = [(b, e) for _, _, b, e in ranges if b < e]
        assert filled and filled[0][0] == first and filled[-1][1] == context
        assert all(a[1] == b[0] and b[0] % KEY_ALIGN == 0 for a, b in zip(filled, filled[1:]))
        assert [(b, e) for _, _, b, e in ranges][len(filled):] == [(context, context)] * (per_tile - len(filled))


@pytest.mark.parametrize("seed", range(10))
def test_plan_of_portions_whose_key_ranges_are_merged_in_the_workgroup(seed):
    """Rows of several tokens: every tile of every row gets four neighbouring items (its key ranges, the last ones may be
    empty) without slots or merges; the ranges of a tile follow one another from the first key its first token may see to
    its last token, at multiples of KEY_ALIGN; filled up to a number of tiles, the arrays have that shape and the
    additions repeat the first tile."""
    rng = random.Random(seed)
    rows = rng.randint(1, 6)
    lens = [rng.choice((1, 2, 7, 8, 9, 40, 128)) for _ in range(rows)]
    contexts = [n + rng.choice((0, 0, 5, 64, 300)) for n in lens]
    window = rng.choice((None, None, 40))
    group_size, n_kv = rng.choice((1, 2, 4, 20)), rng.choice((1, 8))
    if all(n == 1 for n in lens):
        lens[0], contexts[0] = 3, contexts[0] + 2
    _, tokens_per_tile, _ = group_tiling(group_size)
    real = sum(-(-n // tokens_per_tile) for n in lens)
    fixed_tiles = rng.choice((None, real, real + 3))
    plan = build_attention_plan(lens, contexts, group_size, n_kv, window, merge_in_workgroup=4, workgroup_tiles=8, fixed_tiles=fixed_tiles,
                                **({"fixed_splits": 4} if fixed_tiles else {}))
    tiles = fixed_tiles or real
    assert plan.merge_in_workgroup == 4 and plan.items.shape == (4 * tiles, 4) and plan.n_slots == 0 and plan.merges.shape == (0, 4)
    assert (plan.item_slot == -1).all() and plan.tiles.shape == (0, 4) and plan.tile_slots is None
    at = 0
    for row, (n, context) in enumerate(zip(lens, contexts)):
        for q0 in range(0, n, tokens_per_tile):
            ranges = plan.items[4 * at:4 * at + 4].tolist()
            at += 1
            assert all(r == row and q == q0 for r, q, _, _ in ranges)
            last = context - n + min(q0 + tokens_per_tile, n)                # one past the last key the tile's last token sees
            first = 0 if window is None else max(0, context - n + q0 - window + 1)
            filled = [(b, e) for _, _, b, e in ranges if b < e]
            assert filled and filled[0][0] == first and filled[-1][1] == last
            assert all(a[1] == b[0] and b[0] % KEY_ALIGN == 0 for a, b in zip(filled, filled[1:]))
            assert [(b, e) for _, _, b, e in ranges][len(filled):] == [(last, last)] * (4 - len(filled))
    assert at == real
    for extra in range(real, tiles):                                         # the filling repeats the first tile
        assert (plan.items[4 * extra:4 * extra + 4] == plan.items[:4]).all()
    with pytest.raises(ValueError):                                          # two ranges a tile: single tokens only
        build_attention_plan(lens, contexts, group_size, n_kv, window, merge_in_workgroup=2)


def test_four_or_eight_tiles_per_workgroup_whole_or_in_halves():
    """With the costs measured on an MI355X: one prompt is bounded by its longest workgroup, whose walk two halves
    shorten (eight tiles at 2,048 tokens, four below); long rows and many rows keep every compute unit busy and take eight
    tiles and no halves; a kernel that offers only four tiles, or no halves, gets what it offers."""
    from llmserver_amd.parts import AttentionTuning, TileLaunchCost
    tuning = AttentionTuning(1024, (((False, 1), TileLaunchCost(3.2, 1.16, 2.0)), ((True, 1), TileLaunchCost(8.7, 1.16, 2.75)),
                                    ((False, 2), TileLaunchCost(3.3, 1.7, 2.42)), ((True, 2), TileLaunchCost(8.8, 1.7, 3.38))))

    def chosen(lens, ctxs, most=8, halves=2):
        plan = build_attention_plan(lens, ctxs, 4, 8, None, workgroup_tiles=most, tuning=tuning, tile_halves=halves)
        return plan.tiles_per_workgroup, plan.tile_halves
    assert chosen([2048], [2048]) == (8, 2)
    assert chosen([1024], [1024]) == (4, 2)
    assert chosen([512], [2560]) == (4, 2)                                   # a portion behind a prefix
    assert chosen([4096], [4096]) == (8, 1)
    assert chosen([2048], [32768]) == (8, 1)
    assert chosen([512] * 16, [512] * 16) == (8, 1)
    assert chosen([1024], [1024], halves=1) == (4, 1)                        # a kernel without halves
    assert chosen([4096], [4096], most=4) == (4, 1)
    assert chosen([1] * 8, [4096] * 8) == (0, 1)                             # no row has enough tiles
    assert build_attention_plan([4096], [4096], 4, 8, None).tiles_per_workgroup == 0
    # a kernel that needs many workgroups to pay gets them or nothing
    few = build_attention_plan([512], [2560], 4, 8, None, workgroup_tiles=4, tile_min_workgroups=512)
    many = build_attention_plan([2048], [2048], 4, 8, None, workgroup_tiles=4, tile_min_workgroups=512)
    assert (few.tiles_per_workgroup, len(few.tiles)) == (0, 0) and len(few.items) == 128
    assert (many.tiles_per_workgroup, len(many.tiles)) == (4, 128)


def test_short_rows_behind_long_contexts_share_their_keys_between_workgroups():
    """With the costs measured on an MI355X and a kernel that offers key ranges: a portion of 64 tokens behind 4,032 is
    cut into ranges of at most 16 steps for workgroups of their own (four workgroups a KV head would otherwise walk 128
    steps each), eight rows of 16 tokens likewise, rows of 8 tokens go to that kernel at all; a whole prompt is not cut;
    beside a whole prompt only the short row is."""
    from llmserver_amd.parts import AttentionTuning, TileLaunchCost
    tuning = AttentionTuning(1024, (((False, 1), TileLaunchCost(3.2, 0.89, 1.55)), ((True, 1), TileLaunchCost(8.7, 0.94, 2.45)),
                                    ((False, 2), TileLaunchCost(3.3, 1.11, 2.08)), ((True, 2), TileLaunchCost(8.8, 1.44, 2.84))))

    def plan_of(lens, ctxs, key_ranges=128):
        return build_attention_plan(lens, ctxs, 4, 8, None, workgroup_tiles=8, tuning=tuning, tile_halves=2, tile_key_ranges=key_ranges)
    plan = plan_of([64], [4096])
    assert len(plan.items) == 0 and plan.tile_slots is not None and len(plan.merges) == 16 and int(plan.merges[:, 3].min()) >= 4
    steps = -(-(plan.tiles[:, 3] - plan.tiles[:, 2]) // 32)
    assert int(steps.max()) * (1 if plan.tile_halves == 2 else 2) <= 32
    plan = plan_of([16] * 8, [4096] * 8)
    assert len(plan.items) == 0 and plan.tile_slots is not None and len(plan.merges) == 32
    plan = plan_of([8] * 32, [512] * 32)
    assert len(plan.items) == 0 and len(plan.tiles) == 32 and plan.tile_slots is None and plan.n_slots == 0
    plan = plan_of([2048], [2048])
    assert plan.tile_slots is None and plan.n_slots == 0 and (plan.tiles_per_workgroup, plan.tile_halves) == (8, 2)
    plan = plan_of([2048, 64], [2048, 4096])
    with_slots = plan.tiles[plan.tile_slots[:, 0] >= 0]
    assert len(with_slots) and (with_slots[:, 0] == 1).all()
    # a kernel that offers no ranges keeps short rows out (they would be a few workgroups' long walk) and cuts nothing
    plan = plan_of([64, 40], [4096, 4096], key_ranges=1)
    assert plan.tile_slots is None and {int(r) for r in plan.tiles[:, 0]} == {0} and {int(r) for r in plan.items[:, 0]} == {1}
    # decoded tokens never go there
    plan = plan_of([1] * 8 + [64], [4096] * 9)
    assert {int(r) for r in plan.items[:, 0]} == set(range(8)) and {int(r) for r in plan.tiles[:, 0]} == {8}
    # and a handful of tiles stays beside them: no launch of its own, and no merge, for two tiles
    plan = plan_of([1] * 8 + [8], [4096] * 9)
    assert len(plan.tiles) == 0 and {int(r) for r in plan.items[:, 0]} == set(range(9))
