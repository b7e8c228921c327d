"""Grouped-query causal attention over a paged cache, with optional per-head q/k RMSNorm,
rotate-half position encoding and an optional window.

Formulas in execution order (utils/attention.py:114-160, 183-197):
``q,k,v = x Wq^T, x Wk^T, x Wv^T`` as one stacked product (54-66, 124-126); per head
``q^ = q * rsqrt(mean_d(q^2) + eps) * w_q`` and the same for k, before the rotation (157-158;
fused form utils/fused_ops.py:90-134); rotation of q and k by the absolute
position; rotated k and raw v of every new token go to the cache before attention reads it
(utils/kv_cache.py:335-349), so a token sees itself; query head ``h`` uses KV head
``h // G`` (utils/attention.py:77,188); scores ``q.k * scale`` with
``scale = head_dim^-0.5`` by default (utils/architecture.py:105), causal within
the request, softmax and accumulation in 32-bit (utils/attention.py:75-96,197);
output projection (299-300).

The attention kernel works through a list of work items made on the host once a step
(:func:`build_attention_plan`): an item is 16 rows of (token, head-of-the-group) pairs against
a contiguous range of keys.  Rows with few tokens and many keys are cut into several items
whose partial results a second kernel merges by log-sum-exp, the reference's split-KV idea
(utils/paged_attention.py:78-115).
"""
from __future__ import annotations

import dataclasses
from typing import Optional, Tuple

import numpy as np

from .base import VECTOR, Mixer, PagedKVSpec, ParamSpec, PositionEncoding
from .kernel_namespace import tuning_of
from .linear import Linear

# Neutral defaults of the plan's geometry (AttentionTuning carries them; a kernel namespace may say otherwise per type):
TILE_ROWS = 16          # rows of (token, group head) pairs that one work item handles
KEY_ALIGN = 32          # key ranges of split items start at multiples of this
KEY_STEP = 32           # keys that a workgroup of the prompt-portion kernel takes per trip through its loop
MAX_SPLITS = 128        # key ranges per tile (what the kernel that merges them takes, which the kernel namespace checks)
MIN_KEYS_PER_SPLIT = 64     # shorter key ranges than this are not worth a work item of their own
TILE_WALKS = (512, 256, 128, 64, 32, 16, 8)      # most steps a workgroup may be left with, if its keys are cut


@dataclasses.dataclass(frozen=True)
class TileLaunchCost:
    """What one way of launching the prompt-portion kernel costs: microseconds of start and end, microseconds of one
    trip of a workgroup through its loop (``key_step`` keys; a workgroup makes its trips one after the other, so its
    longest workgroup bounds a launch), and nanoseconds of one such step of one workgroup per KV head when every compute
    unit is busy (the work of all workgroups together bounds a launch, too)."""
    start_us: float = 4.0
    trip_us: float = 1.0
    step_ns: float = 1.0


@dataclasses.dataclass(frozen=True)
class AttentionTuning:
    """What the plan needs to know of the machine and its kernels; the kernel namespace of a step supplies it
    (``ops.attention_tuning``), these defaults stand where it does not.

    ``target_waves``: wavefronts wanted in flight; rows with few tokens and long contexts are cut into key ranges
    until there are about that many.  ``tile_costs``: the prompt-portion kernel's workgroups take four tiles or the
    most the kernel offers, and walk their keys whole or in two halves side by side; the costs of each of these
    ways, keyed by (takes the most tiles, halves).  Where the kernel can give ranges of a workgroup's keys to
    workgroups of their own, the partial results cost ``merge_us`` and ``slot_ns``, and rows need only
    ``min_tiles_with_ranges`` tiles to go there (without ranges, a short row behind a long context would be a few
    workgroups' long walk).

    The geometry of the kernels' work items stands here, too, so that the plan is cut for the kernels that will run it:
    ``tile_rows`` (token, head) pairs to an item, key ranges that begin at multiples of ``key_align`` keys, at most
    ``most_splits`` of them to a tile and none shorter than ``fewest_keys_per_split`` (but the last), ``key_step`` keys
    per trip of the prompt-portion kernel, and the walks (in steps) that its workgroups' keys may be cut down to."""
    target_waves: int = 1024
    tile_costs: Tuple[Tuple[Tuple[bool, int], TileLaunchCost], ...] = (
        ((False, 1), TileLaunchCost()), ((True, 1), TileLaunchCost()), ((False, 2), TileLaunchCost()), ((True, 2), TileLaunchCost()))
    merge_us: float = 4.0               # a launch that merges partial results, and ...
    slot_ns: float = 8.0                # ... writing and reading one tile's partial result of one key range, per KV head
    min_tiles_with_ranges: int = 2      # rows with this many tiles go to the prompt-portion kernel if it can cut their keys
                                        # (and if such rows have MIN_TILES_FOR_WORKGROUPS tiles together)
    tile_rows: int = TILE_ROWS
    key_align: int = KEY_ALIGN
    key_step: int = KEY_STEP
    most_splits: int = MAX_SPLITS
    fewest_keys_per_split: int = MIN_KEYS_PER_SPLIT
    tile_walks: Tuple[int, ...] = TILE_WALKS

    def tile_cost(self, takes_most: bool, halves: int) -> TileLaunchCost:
        return dict(self.tile_costs).get((bool(takes_most), int(halves)), TileLaunchCost())


DEFAULT_TUNING = AttentionTuning()
TARGET_WAVES = DEFAULT_TUNING.target_waves


@dataclasses.dataclass(frozen=True)
class AttentionNames:
    """Checkpoint names of an attention layer's tensors, relative to the layer.  ``qkv`` lists the tensors whose rows,
    stacked in this order, are the query, key and value projections: three tensors, two (queries; keys and values
    together) or one that holds all three.  The defaults are the names most decoder checkpoints use."""
    qkv: Tuple[str, ...] = ("q_proj", "k_proj", "v_proj")
    out: str = "o_proj"
    q_norm: str = "q_norm"
    k_norm: str = "k_norm"


def group_tiling(group_size: int, tile_rows: int = TILE_ROWS):
    """(heads of a group per tile, tokens per tile, tiles needed to cover the group)."""
    heads = min(group_size, tile_rows)
    return heads, tile_rows // heads, -(-group_size // heads)


class AttentionPlan:
    """Host arrays of one step's attention work.

    ``items [n_items, 4] int32``: row, first token of the tile within the row's portion, first
    key, one past the last key.  ``item_slot [n_items] int32``: index of the partial-result slot,
    or -1 if the item covers all keys of its rows and writes the output itself.
    ``merges [n_merges, 4] int32``: row, first token of the tile, first slot, number of slots.
    ``tiles [n_tiles, 4] int32``: row, first token, first key, one past the last key of
    ``tiles_per_workgroup`` (4 or 8) consecutive tiles that one workgroup handles together, sharing
    the keys it loads (in ``tile_halves`` halves of its wavefronts, each on its share of the keys).
    ``tile_slots [n_tiles, 2] int32`` or None: where the keys of some workgroups' tiles are cut into ranges, each range
    an entry of ``tiles`` of its own, the first slot of the entry's partial results and the slots between one of its
    tiles and the next (tile j writes slot first + j * stride); first = -1: the entry has all keys and writes the
    output.  ``merges`` holds the merges of such tiles, too.
    """

    def __init__(self, items, item_slot, merges, n_slots, tiles=None, tiles_per_workgroup=0, tile_halves=1, tile_slots=None):
        self.items, self.item_slot, self.merges, self.n_slots = items, item_slot, merges, n_slots
        self.tiles = tiles if tiles is not None else np.zeros((0, 4), dtype=np.int32)
        self.tile_slots = tile_slots
        self.tiles_per_workgroup = tiles_per_workgroup
        self.tile_halves = tile_halves       # 2: the workgroups of ``tiles`` walk their keys in two halves side by side
        self.merge_in_workgroup = 0          # 4: items 4 i .. 4 i + 3 are one tile's key ranges, merged by their workgroup;
                                             # 2: they are the two ranges of each of two tiles


def fixed_split_count(n_rows: int, group_size: int, n_kv_heads: int, max_keys: int, target_waves: int = TARGET_WAVES,
                      tuning: AttentionTuning = DEFAULT_TUNING) -> int:
    """Splits per row when the plan's shape must not depend on the rows' contexts (a captured
    graph of a decode step): enough to fill the chip, never pieces shorter than ``fewest_keys_per_split``
    at the longest context the graph serves."""
    _, _, group_tiles = group_tiling(group_size, tuning.tile_rows)
    waves = max(1, n_rows * n_kv_heads * group_tiles)
    return max(1, min(tuning.most_splits, target_waves // waves, max_keys // tuning.fewest_keys_per_split))


MIN_TILES_FOR_WORKGROUPS = 16      # rows with at least this many tiles go to the prompt-portion kernel (see AttentionTuning for rows with fewer)



def _ranges_of_steps(steps, walk, most_ranges):
    """Into how many ranges ``steps`` steps of keys are cut when no workgroup is to walk more than ``walk``."""
    if walk is None or most_ranges <= 1:
        return np.ones_like(steps)
    return np.minimum(most_ranges, np.maximum(1, -(-steps // walk)))


def _workgroups_of_rows(rows, row_len, row_ctx, tokens_per_tile, window, per_workgroup):
    """The workgroups that ``rows`` make with ``per_workgroup`` tiles each, all rows at once: arrays of their row, first
    token, first key, one past the last key, and tiles (the last workgroup of a row may have fewer)."""
    lens = row_len[rows]
    first_positions = row_ctx[rows] - lens
    span = per_workgroup * tokens_per_tile
    groups_of_row = -(-lens // span)
    of_row = np.repeat(np.arange(len(rows)), groups_of_row)
    starts = (np.arange(int(groups_of_row.sum())) - np.repeat(np.cumsum(groups_of_row) - groups_of_row, groups_of_row)) * span
    k_end = first_positions[of_row] + np.minimum(starts + span, lens[of_row])
    k_begin = np.zeros_like(starts) if window is None else np.maximum(0, first_positions[of_row] + starts - window + 1)
    tiles = -(-np.minimum(span, lens[of_row] - starts) // tokens_per_tile)
    return rows[of_row], starts, k_begin, k_end, tiles


def _workgroup_tiles_that_pay(row_len, row_ctx, tiles_per_row, tokens_per_tile, heads, window, most: int,
                              tuning: AttentionTuning = DEFAULT_TUNING, most_halves: int = 1, most_ranges: int = 1,
                              min_tiles: int = MIN_TILES_FOR_WORKGROUPS, workgroups: Optional[dict] = None):
    """``(tiles per workgroup, halves, walk)`` of the prompt-portion kernel that the step's rows finish soonest with:
    4 or ``most`` tiles, the keys of a workgroup walked whole or, where the kernel can, in two halves side by side,
    and, where the kernel can (``most_ranges`` > 1), cut into ranges of at most ``walk`` steps for workgroups of
    their own (None: never cut).

    A workgroup walks its keys in steps of ``tuning.key_step``.  More tiles per workgroup get more out of every step (setting up and
    draining a workgroup costs about 8 steps more), and two halves halve the trips of the longest workgroup, which
    bounds a launch of few workgroups from below; but steps of larger workgroups take longer, which is what counts
    when every compute unit is busy.  Ranges shorten the longest walk as far as one likes, for the price of a
    second launch and the partial results' way through memory.  Each way is priced with the tuning's costs: start,
    then the longest workgroup's trips and all workgroups' steps, whichever is more (blended, since both slow each
    other down), then the merge.  Shorter and shorter walks are priced until one costs more than the one before."""
    rows = np.flatnonzero(np.asarray(tiles_per_row) >= min_tiles)
    row_len, row_ctx = np.asarray(row_len, dtype=np.int64), np.asarray(row_ctx, dtype=np.int64)
    best, best_key = None, None
    for per_workgroup in sorted({min(4, most), most}):
        of_rows = _workgroups_of_rows(rows, row_len, row_ctx, tokens_per_tile, window, per_workgroup)
        if workgroups is not None:
            workgroups[per_workgroup] = of_rows                  # (the caller goes on with those of the way chosen)
        _, _, k_begin, k_end, tiles_of_group = of_rows
        steps = -(-(k_end - k_begin) // tuning.key_step)
        unsplit = int(steps.max(initial=0))
        for halves in sorted({1, max(1, int(most_halves))}):
            cost = tuning.tile_cost(per_workgroup > 4, halves)
            before = None
            for walk in (None,) + (tuple(w for w in tuning.tile_walks if w < unsplit) if most_ranges > 1 else ()):
                if walk is None:
                    total, longest, slots = int(steps.sum()) + 8 * len(steps), unsplit, 0
                else:
                    ranges = _ranges_of_steps(steps, walk, most_ranges)
                    per_range = -(-steps // ranges)
                    total = int((per_range * ranges).sum()) + 8 * int(ranges.sum())
                    longest = int(per_range.max(initial=0))
                    slots = int((ranges * tiles_of_group)[ranges > 1].sum())
                path, work = -(-longest // halves) * cost.trip_us, total * heads * cost.step_ns * 1e-3
                merge = tuning.merge_us + slots * heads * tuning.slot_ns * 1e-3 if slots else 0.0
                estimate = cost.start_us + (path ** 4 + work ** 4) ** 0.25 + merge
                key = (estimate, walk is not None, halves, per_workgroup)
                if best_key is None or key < best_key:
                    best, best_key = (per_workgroup, halves, walk), key
                if walk is not None and before is not None and estimate > before:
                    break
                before = estimate if walk is not None else before
    return best


WORKGROUP_RANGES = 4    # key ranges of a tile that one workgroup (four wavefronts) walks and merges itself
SHORT_CONTEXT = 512     # captured steps whose contexts all stay within this are a shape of their own: a workgroup merges
                        # a tile's four key ranges itself (no partial results in memory, no launch that merges them)


def _single_token_plan(row_ctx: np.ndarray, window: Optional[int], splits: int, merge_in_workgroup: int = 0,
                       key_align: int = KEY_ALIGN) -> AttentionPlan:
    """The plan of a step in which every row brings one token and every tile gets ``splits`` key ranges: what the
    loop of :func:`build_attention_plan` makes for it, row by row, computed for all rows at once (a decode step of
    many rows is planned thousands of times a second)."""
    n_rows = len(row_ctx)
    rows = np.arange(n_rows, dtype=np.int64)
    k_end = row_ctx
    k_begin = np.zeros_like(k_end) if window is None else np.maximum(0, k_end - window)
    zeros = np.zeros_like(rows)
    if splits <= 1 and not merge_in_workgroup:
        items = np.stack([rows, zeros, k_begin, k_end], axis=1).astype(np.int32)
        return AttentionPlan(items, np.full(n_rows, -1, dtype=np.int32), np.zeros((0, 4), dtype=np.int32), 0)
    if merge_in_workgroup:          # four (or two) items a tile; with fewer ranges wanted, the last ones come out empty
        ranges, splits = max(1, min(splits, merge_in_workgroup)), merge_in_workgroup
    start = (k_begin // key_align) * key_align
    per = -(-(k_end - start) // (ranges if merge_in_workgroup else splits))
    per = -(-per // key_align) * key_align
    piece = start[:, None] + np.arange(splits, dtype=np.int64)[None, :] * per[:, None]
    lo = np.maximum(piece, k_begin[:, None])
    hi = np.minimum(piece + per[:, None], k_end[:, None])
    inside = lo < k_end[:, None]
    first = np.where(inside, lo, k_end[:, None])
    last = np.where(inside, np.maximum(lo, hi), k_end[:, None])
    items = np.stack([np.repeat(rows, splits), np.zeros(n_rows * splits, dtype=np.int64), first.reshape(-1), last.reshape(-1)],
                     axis=1).astype(np.int32)
    if merge_in_workgroup:          # the four items of a tile are one workgroup's: no slots, nothing left to merge
        plan = AttentionPlan(items, np.full(n_rows * splits, -1, dtype=np.int32), np.zeros((0, 4), dtype=np.int32), 0)
        plan.merge_in_workgroup = merge_in_workgroup
        return plan
    merges = np.stack([rows, zeros, rows * splits, np.full(n_rows, splits, dtype=np.int64)], axis=1).astype(np.int32)
    return AttentionPlan(items, np.arange(n_rows * splits, dtype=np.int32), merges, n_rows * splits)


def build_attention_plan(row_len, row_ctx, group_size: int, n_kv_heads: int, window: Optional[int] = None,
                         target_waves: int = TARGET_WAVES, fixed_splits: Optional[int] = None,
                         workgroup_tiles: int = 0, single_token_shortcut: bool = True, merge_in_workgroup: int = 0,
                         tuning: AttentionTuning = DEFAULT_TUNING, tile_halves: int = 1, tile_min_workgroups: int = 0,
                         tile_key_ranges: int = 1, fixed_tiles: Optional[int] = None) -> AttentionPlan:
    """Cut the step's rows into tiles of tokens and, where that pays, ranges of keys.

    With ``fixed_splits`` every tile gets exactly that many items (some may be empty), so the
    arrays have the same shape whatever the contexts are.  With ``workgroup_tiles`` (the number of tiles a
    workgroup of that kernel takes, which the kernel library tells) rows with many tiles (portions of prompts) go
    to the kernel in which the tiles of a workgroup share the keys they load; ``tile_halves`` says whether that kernel
    can split a workgroup's keys between two halves of its wavefronts (2) or not (1), ``tile_min_workgroups`` how many
    workgroups a launch of it needs to be worth while (a kernel whose steps are slow is bounded by its longest
    workgroup unless there are many), ``tile_key_ranges`` into how many ranges it lets the keys of a workgroup's tiles
    be cut, each for a workgroup of its own (1: it does not; more: rows of few tiles go to it as well, and their
    partial results are merged like those of split items).  ``fixed_tiles`` (with ``fixed_splits``): the arrays are
    filled up to the shape of that many tiles, whatever the rows' lengths are (a captured step of prompt portions:
    ``fixed_tiles`` is at least the number of tiles any rows of the step's shape can have), with repetitions of the
    first tile's entries, which compute and write the same numbers once more.  ``merge_in_workgroup`` (4, or 2 in steps
    of one token per row with an even number of rows): every tile gets that many ranges, the items of a workgroup, which
    merges them itself: no slots, no merges, no workgroups of tiles."""
    _, tokens_per_tile, group_tiles = group_tiling(group_size, tuning.tile_rows)
    key_align, key_step, most_splits = tuning.key_align, tuning.key_step, tuning.most_splits
    row_len = np.asarray(row_len, dtype=np.int64)
    row_ctx = np.asarray(row_ctx, dtype=np.int64)
    merge_in_workgroup = WORKGROUP_RANGES if merge_in_workgroup is True else int(merge_in_workgroup)
    single_tokens = bool(len(row_len)) and int(row_len.min()) == 1 == int(row_len.max())
    if merge_in_workgroup == 2 and not single_tokens:
        raise ValueError("two key ranges of each of two tiles are merged in a workgroup only in steps of one token per row")
    if merge_in_workgroup not in (0, 2, WORKGROUP_RANGES) or (merge_in_workgroup == 2 and len(row_len) % 2):
        raise ValueError("a workgroup merges four key ranges of one tile, or two ranges of each of two tiles (an even number of rows)")
    if (merge_in_workgroup or (single_token_shortcut and fixed_splits is not None)) and single_tokens:
        return _single_token_plan(row_ctx, window, int(fixed_splits or merge_in_workgroup or 1), merge_in_workgroup, key_align)
    if merge_in_workgroup:
        # Rows of several tokens: every tile of every row gets exactly four ranges (the last ones may be empty), four
        # neighbouring items, which their workgroup merges: no slots, no merge, and no workgroups of tiles.
        fixed_splits, workgroup_tiles = merge_in_workgroup, 0
    tiles_per_row = -(-row_len // tokens_per_tile)
    waves_unsplit = int(tiles_per_row.sum()) * n_kv_heads * group_tiles
    items, slots, merges, tiles = [], [], [], []
    n_slots = 0
    per_workgroup, halves, walk = 0, 1, None
    workgroups = {}
    most_ranges = max(1, min(int(tile_key_ranges), most_splits))
    min_tiles = tuning.min_tiles_with_ranges if most_ranges > 1 else MIN_TILES_FOR_WORKGROUPS
    # (rows of few tiles go there only if together they have as many as one row needs without ranges: a launch of its
    # own, and a merge, for a handful of tiles costs more than the items they would be beside the step's other rows)
    if workgroup_tiles and fixed_splits is None and int(tiles_per_row[tiles_per_row >= min_tiles].sum()) >= MIN_TILES_FOR_WORKGROUPS:
        per_workgroup, halves, walk = _workgroup_tiles_that_pay(
            row_len, row_ctx, tiles_per_row, tokens_per_tile, n_kv_heads * group_tiles, window, int(workgroup_tiles), tuning,
            int(tile_halves), most_ranges, min_tiles, workgroups=workgroups)
        if per_workgroup and tile_min_workgroups:
            groups = sum(-(-int(n) // (per_workgroup * tokens_per_tile)) for n, tiles_of_row in zip(row_len, tiles_per_row)
                         if tiles_of_row >= min_tiles)
            if groups * n_kv_heads * group_tiles < tile_min_workgroups:
                per_workgroup, halves = 0, 1
    if per_workgroup:
        # The rows of many tiles, all at once: a workgroup for every ``per_workgroup`` tiles, or one for each range of
        # their keys.  Tile j of a workgroup whose keys are cut leaves the partial result of range s in slot
        # first + j * ranges + s, where ``first`` is the group's first slot.
        rows_in_tiles = np.flatnonzero(tiles_per_row >= min_tiles)
        of_row, starts, k_begin, k_end, tiles_of_group = workgroups.get(per_workgroup) or _workgroups_of_rows(
            rows_in_tiles, row_len, row_ctx, tokens_per_tile, window, per_workgroup)
        aligned = (k_begin // key_align) * key_align
        steps = -(-(k_end - aligned) // key_step)
        per = -(-steps // _ranges_of_steps(steps, walk, most_ranges)) * key_step
        per = -(-per // key_align) * key_align                                          # (ranges begin at multiples of key_align)
        ranges = np.maximum(1, -(-(k_end - aligned) // np.maximum(per, key_align)))      # (none of them empty)
        cut = ranges > 1
        first = np.cumsum(np.where(cut, ranges * tiles_of_group, 0)) - np.where(cut, ranges * tiles_of_group, 0)
        n_slots = int(np.where(cut, ranges * tiles_of_group, 0).sum())
        group = np.repeat(np.arange(len(ranges)), ranges)                        # an entry for every range of every group
        s = np.arange(len(group)) - np.repeat(np.cumsum(ranges) - ranges, ranges)
        entry_begin = np.maximum(k_begin[group], aligned[group] + s * per[group])
        entry_end = np.minimum(k_end[group], aligned[group] + (s + 1) * per[group])
        tiles = np.stack([of_row[group], starts[group], entry_begin, entry_end,
                          np.where(cut[group], first[group] + s, -1), np.where(cut[group], ranges[group], 0)], axis=1)
        if n_slots:
            cut_groups = np.flatnonzero(cut)
            group = np.repeat(cut_groups, tiles_of_group[cut_groups])            # a merge for every tile of every cut group
            j = np.arange(len(group)) - np.repeat(np.cumsum(tiles_of_group[cut_groups]) - tiles_of_group[cut_groups], tiles_of_group[cut_groups])
            merges = np.stack([of_row[group], starts[group] + j * tokens_per_tile, first[group] + j * ranges[group], ranges[group]], axis=1).tolist()
    for row in range(len(row_len)):
        n, ctx = int(row_len[row]), int(row_ctx[row])
        first_pos = ctx - n
        if per_workgroup and tiles_per_row[row] >= min_tiles:
            continue
        for tile in range(int(tiles_per_row[row])):
            q0 = tile * tokens_per_tile
            q1 = min(q0 + tokens_per_tile, n)
            k_end = first_pos + q1                       # last query of the tile sees keys < k_end
            k_begin = 0 if window is None else max(0, first_pos + q0 - window + 1)
            n_keys = k_end - k_begin
            splits = 1
            if fixed_splits is not None:
                splits = fixed_splits
            elif waves_unsplit < target_waves:
                splits = min(most_splits, max(1, target_waves // max(1, waves_unsplit)), max(1, n_keys // tuning.fewest_keys_per_split))
            if splits <= 1:
                items.append((row, q0, k_begin, k_end))
                slots.append(-1)
                continue
            start = (k_begin // key_align) * key_align
            per = -(-(k_end - start) // splits)
            per = -(-per // key_align) * key_align        # at most `splits` items, each a multiple of key_align keys
            first_slot = n_slots
            count = 0
            while start < k_end or (fixed_splits is not None and count < splits):
                lo, hi = max(start, k_begin), min(start + per, k_end)
                items.append((row, q0, lo, max(lo, hi)) if lo < k_end else (row, q0, k_end, k_end))
                slots.append(-1 if merge_in_workgroup else n_slots)
                n_slots += 0 if merge_in_workgroup else 1
                count += 1
                start += per
            if not merge_in_workgroup:
                merges.append((row, q0, first_slot, count))
    if fixed_tiles is not None:
        if fixed_splits is None or len(tiles):
            raise ValueError("a plan is filled up to a number of tiles only where every tile gets a fixed number of key ranges")
        real = len(items) // fixed_splits
        if real < 1 or real > fixed_tiles:
            raise ValueError(f"the step's rows make {real} tiles, the shape it is filled up to holds {fixed_tiles}")
        items += items[:fixed_splits] * (fixed_tiles - real)
        slots += slots[:fixed_splits] * (fixed_tiles - real)
        merges += merges[:1] * (fixed_tiles - real)
        n_slots = fixed_tiles * fixed_splits if merges else 0
    items = np.asarray(items, dtype=np.int32).reshape(-1, 4)
    merges = np.asarray(merges, dtype=np.int32).reshape(-1, 4)
    tiles = np.asarray(tiles, dtype=np.int32).reshape(-1, 6)
    tiles = tiles[np.argsort(tiles[:, 2] - tiles[:, 3], kind="stable")]       # most keys first: the long tiles must not start last
    tile_slots = np.ascontiguousarray(tiles[:, 4:]) if len(tiles) and int(tiles[:, 4].max()) >= 0 else None
    plan = AttentionPlan(items, np.asarray(slots, dtype=np.int32), merges, n_slots, np.ascontiguousarray(tiles[:, :4]),
                         per_workgroup if len(tiles) else 0, halves if len(tiles) else 1, tile_slots)
    plan.merge_in_workgroup = merge_in_workgroup
    return plan


class GQAttention(Mixer):
    graph_safe = True
    accepts_pending_norm = True
    takes_sink = True

    def __init__(self, width: int, n_heads: int, n_kv_heads: int, head_dim: int, position: PositionEncoding,
                 qk_norm_eps: Optional[float] = None, bias: bool = False, out_bias: Optional[bool] = None,
                 window: Optional[int] = None, scale: Optional[float] = None, names: AttentionNames = AttentionNames()):
        if n_heads % n_kv_heads:
            raise ValueError(f"Number of query heads must be divisible by the number of KV heads: query heads: {n_heads}, KV heads: {n_kv_heads}")
        self.width, self.n_heads, self.n_kv_heads, self.head_dim = width, n_heads, n_kv_heads, head_dim
        self.group_size = n_heads // n_kv_heads
        if position.rotary_dim is not None and position.rotary_dim != head_dim:
            raise ValueError(f"the position encoding rotates {position.rotary_dim} of a head's {head_dim} dimensions; this mixer's "
                             "kernels rotate the whole head or nothing (a rotation of a part of the head is not built)")
        self.position = position
        self.qk_norm_eps = qk_norm_eps
        self.window = window
        self.scale = float(scale) if scale is not None else float(head_dim) ** -0.5
        q_rows, kv_rows = n_heads * head_dim, n_kv_heads * head_dim
        stacked = {3: (q_rows, kv_rows, kv_rows), 2: (q_rows, 2 * kv_rows), 1: (q_rows + 2 * kv_rows,)}
        if len(names.qkv) not in stacked:
            raise ValueError(f"queries, keys and values come in one, two or three checkpoint tensors, not {len(names.qkv)}")
        self.names = names
        self.qkv = Linear(width, names.qkv, stacked[len(names.qkv)], bias)
        self.o = Linear(q_rows, (names.out,), (width,), bias if out_bias is None else out_bias)
        self.q_norm_weight = None
        self.k_norm_weight = None

    def cache_spec(self):
        return PagedKVSpec(self.n_kv_heads, self.head_dim, self.window)

    def param_specs(self):
        specs = {**self.qkv.param_specs(), **self.o.param_specs()}
        if self.qk_norm_eps is not None:
            specs[f"{self.names.q_norm}.weight"] = ParamSpec((self.head_dim,), VECTOR, "norm")
            specs[f"{self.names.k_norm}.weight"] = ParamSpec((self.head_dim,), VECTOR, "norm")
        return specs

    def assign(self, name, tensor):
        owner = name.rsplit(".", 1)[0]
        if owner == self.names.q_norm:
            self.q_norm_weight = tensor
        elif owner == self.names.k_norm:
            self.k_norm_weight = tensor
        elif owner == self.names.out:
            self.o.assign(name, tensor)
        elif owner in self.names.qkv:
            self.qkv.assign(name, tensor)
        else:
            raise KeyError(name)

    def finalize(self):
        self.qkv.finalize()
        self.o.finalize()

    def plan_key(self):
        return ("paged_attention", self.group_size, self.n_kv_heads, self.window)

    def graph_shape(self, rows: int, longest_context: int):
        return "short contexts" if longest_context <= SHORT_CONTEXT else None

    def graph_shape_edges(self):
        return (SHORT_CONTEXT,)

    def mixing_flops(self, new_tokens: int, context: int) -> float:
        """Scores and weighted values: two products of ``head_dim`` multiply-adds per query head, query and visible key."""
        first = context - new_tokens
        if self.window is None:
            pairs = new_tokens * first + new_tokens * (new_tokens + 1) // 2
        else:
            pairs = sum(min(position + 1, self.window) for position in range(first, context))
        return 4.0 * self.n_heads * self.head_dim * pairs

    def prepare(self, ctx):
        key = self.plan_key()
        if ctx.has_plan(key):
            return
        fixed = fixed_tiles = None
        tuning = tuning_of(ctx.ops, DEFAULT_TUNING, ctx.dtype, self.head_dim)
        single_tokens = ctx.n_tokens == ctx.n_rows
        if ctx.static_max_keys is not None and single_tokens:          # a step whose shapes must not depend on the contexts
            fixed = fixed_split_count(ctx.n_rows, self.group_size, self.n_kv_heads, ctx.static_max_keys, tuning.target_waves, tuning)
        elif ctx.static_max_keys is not None:
            # ... nor on how its tokens are spread over its rows: as many tiles as rows of this many tokens can have at
            # most (a row's last tile may be partly empty), every tile with the same number of key ranges.
            _, tokens_per_tile, _ = group_tiling(self.group_size, tuning.tile_rows)
            fixed_tiles = ctx.n_tokens // tokens_per_tile + ctx.n_rows
            fixed = fixed_split_count(fixed_tiles, self.group_size, self.n_kv_heads, ctx.static_max_keys, tuning.target_waves, tuning)
        # Where a workgroup can merge a tile's key ranges itself, the merge launch and the partial results go:
        #  * short contexts (a shape of captured steps of its own, see graph_shape): four ranges a tile, in steps of
        #    single tokens and in captured steps with portions alike;
        #  * so many rows that a tile gets four ranges anyway;
        #  * two ranges a tile: two tiles to a workgroup, if the rows come in pairs.  (Two or three ranges in a workgroup
        #    of one tile leave wavefronts idle through the others' walk: a tenth slower at 64 rows behind 4,096 tokens.)
        in_workgroup = 0
        if single_tokens:
            if ctx.static_max_keys is not None and self.graph_shape(ctx.n_rows, int(np.max(ctx.h_row_ctx))) is not None:
                in_workgroup = fixed = WORKGROUP_RANGES
            elif fixed == WORKGROUP_RANGES or (fixed == 2 and ctx.n_rows % 2 == 0):
                in_workgroup = fixed
        elif ctx.static_max_keys is not None and self.graph_shape(ctx.n_rows, int(np.max(ctx.h_row_ctx))) is not None:
            in_workgroup = fixed = WORKGROUP_RANGES
        per_workgroup = ctx.ops.attention_workgroup_tiles(ctx.dtype, self.head_dim, ctx.page_size)
        halves = ctx.ops.attention_tile_halves(ctx.dtype, self.head_dim) if per_workgroup else 1
        fewest = ctx.ops.attention_tile_min_workgroups(ctx.dtype) if per_workgroup else 0
        key_ranges = ctx.ops.attention_tile_key_ranges(ctx.dtype, self.head_dim) if per_workgroup else 1
        plan = build_attention_plan(ctx.h_row_len, ctx.h_row_ctx, self.group_size, self.n_kv_heads, self.window,
                                    target_waves=tuning.target_waves, fixed_splits=fixed, workgroup_tiles=per_workgroup,
                                    merge_in_workgroup=in_workgroup, tuning=tuning, tile_halves=halves, tile_min_workgroups=fewest,
                                    tile_key_ranges=key_ranges, fixed_tiles=fixed_tiles)
        ctx.set_plan(key, {
            **({"tile_slots": plan.tile_slots} if plan.tile_slots is not None else {}),
            "items": plan.items, "item_slot": plan.item_slot, "merges": plan.merges, "tiles": plan.tiles,
            "n_tiles": len(plan.tiles), "n_items": len(plan.items), "n_merges": len(plan.merges),
            "n_slots": plan.n_slots, "tiles_per_workgroup": plan.tiles_per_workgroup, "tile_halves": int(plan.tile_halves),
            "merge_in_workgroup": int(plan.merge_in_workgroup),
            "most_splits": int(plan.merges[:, 3].max()) if len(plan.merges) else 0,
        })

    def forward(self, x, ctx, cache, sink=None):
        qkv = self.qkv.forward(x, ctx)
        table = ctx.block_table(cache.group)
        eps = self.qk_norm_eps if self.qk_norm_eps is not None else 0.0
        cos_sin = self.position.cos_sin(ctx)
        # A step of single tokens: the attention kernel does the norm, the rotation and the cache write itself.
        fusion = None
        # (the kernel that merges a tile's key ranges in its workgroup fuses only the whole of norm and rotation)
        whole = self.q_norm_weight is not None and cos_sin is not None
        if ctx.n_tokens == ctx.n_rows and ctx.ops.decode_fusion_fits(qkv.dtype, self.head_dim) \
                and (whole or not ctx.get_plan(self.plan_key()).get("merge_in_workgroup")):
            fusion = (self.q_norm_weight, self.k_norm_weight, eps, cos_sin, cache.writable)
        else:
            ctx.ops.qk_norm_rope_kv_write(
                qkv, cache.keys, cache.values, table, ctx.token_row, ctx.positions, self.q_norm_weight, self.k_norm_weight, eps,
                cos_sin, cache.page_size, self.n_heads, self.n_kv_heads, self.head_dim, cache.writable)
        out = ctx.empty((qkv.shape[0], self.n_heads * self.head_dim))
        extra = {"decode_fusion": fusion} if fusion is not None else {}
        ctx.ops.paged_attention(
            qkv, out, cache.keys, cache.values, table, ctx.row_start, ctx.row_len, ctx.row_ctx,
            ctx.get_plan(self.plan_key()), self.scale, self.window, cache.page_size,
            self.n_heads, self.n_kv_heads, self.head_dim, ctx, **extra)
        return self.o.forward(out, ctx, sink=sink)
