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

TILE_ROWS = 16          # rows of (token, group head) pairs one wavefront handles (MFMA N dimension)
KEY_ALIGN = 32          # key ranges of split items start at multiples of this
MAX_SPLITS = 128        # key ranges per tile (the merge kernel's limit, which the kernel namespace checks)
MIN_KEYS_PER_SPLIT = 64     # shorter key ranges than this are not worth a wavefront of their own


@dataclasses.dataclass(frozen=True)
class TileLaunchCost:
    """What one way of launching the prompt-portion kernel costs: microseconds of start and end, microseconds of one
    trip of a workgroup through its loop (32 keys; a workgroup makes its trips one after the other, so its longest
    workgroup bounds a launch), and nanoseconds of one 32-key step of one workgroup per KV head when every compute
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
    ways, keyed by (takes the most tiles, halves)."""
    target_waves: int = 1024
    tile_costs: Tuple[Tuple[Tuple[bool, int], TileLaunchCost], ...] = (
        ((False, 1), TileLaunchCost()), ((True, 1), TileLaunchCost()), ((False, 2), TileLaunchCost()), ((True, 2), TileLaunchCost()))

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


def group_tiling(group_size: int):
    """(heads of a group per tile, tokens per tile, tiles needed to cover the group)."""
    heads = min(group_size, TILE_ROWS)
    return heads, TILE_ROWS // heads, -(-group_size // heads)


class AttentionPlan:
    """Host arrays of one step's attention work.

    ``items [n_items, 4] int32``: row, first token of the tile within the row's portion, first
    key, one past the last key.  ``item_slot [n_items] int32``: index of the partial-result slot,
    or -1 if the item covers all keys of its rows and writes the output itself.
    ``merges [n_merges, 4] int32``: row, first token of the tile, first slot, number of slots.
    ``tiles [n_tiles, 4] int32``: row, first token, first key, one past the last key of
    ``tiles_per_workgroup`` (4 or 8) consecutive tiles that one workgroup handles together, sharing
    the keys it loads (in ``tile_halves`` halves of its wavefronts, each on its share of the keys).
    """

    def __init__(self, items, item_slot, merges, n_slots, tiles=None, tiles_per_workgroup=0, tile_halves=1):
        self.items, self.item_slot, self.merges, self.n_slots = items, item_slot, merges, n_slots
        self.tiles = tiles if tiles is not None else np.zeros((0, 4), dtype=np.int32)
        self.tiles_per_workgroup = tiles_per_workgroup
        self.tile_halves = tile_halves       # 2: the workgroups of ``tiles`` walk their keys in two halves side by side
        self.merge_in_workgroup = 0          # 4: items 4 i .. 4 i + 3 are one tile's key ranges, merged by their workgroup;
                                             # 2: they are the two ranges of each of two tiles


def fixed_split_count(n_rows: int, group_size: int, n_kv_heads: int, max_keys: int, target_waves: int = TARGET_WAVES) -> int:
    """Splits per row when the plan's shape must not depend on the rows' contexts (a captured
    graph of a decode step): enough to fill the chip, never pieces shorter than MIN_KEYS_PER_SPLIT
    at the longest context the graph serves."""
    _, _, group_tiles = group_tiling(group_size)
    waves = max(1, n_rows * n_kv_heads * group_tiles)
    return max(1, min(MAX_SPLITS, target_waves // waves, max_keys // MIN_KEYS_PER_SPLIT))


MIN_TILES_FOR_WORKGROUPS = 16      # rows with at least this many tiles go to the prompt-portion kernel


def _workgroup_tiles_that_pay(row_len, row_ctx, tiles_per_row, tokens_per_tile, heads, window, most: int,
                              tuning: AttentionTuning = DEFAULT_TUNING, most_halves: int = 1):
    """``(tiles per workgroup, halves)`` of the prompt-portion kernel that the step's rows finish soonest with: 4 or
    ``most`` tiles, the keys of a workgroup walked whole or, where the kernel can, in two halves side by side.

    A workgroup walks its keys in steps of 32.  More tiles per workgroup get more out of every step (setting up and
    draining a workgroup costs about 8 steps more), and two halves halve the trips of the longest workgroup, which
    bounds a launch of few workgroups from below; but steps of larger workgroups take longer, which is what counts
    when every compute unit is busy.  Each way is priced with the tuning's costs: start, then the longest
    workgroup's trips and all workgroups' steps, whichever is more (blended, since both slow each other down)."""
    def estimate(per_workgroup, halves):
        cost = tuning.tile_cost(per_workgroup > 4, halves)
        span = per_workgroup * tokens_per_tile
        total = longest = 0
        for row in range(len(row_len)):
            if tiles_per_row[row] < MIN_TILES_FOR_WORKGROUPS:
                continue
            n, first_pos = int(row_len[row]), int(row_ctx[row]) - int(row_len[row])
            starts = np.arange(0, n, span)
            k_end = first_pos + np.minimum(starts + span, n)
            k_begin = np.zeros_like(starts) if window is None else np.maximum(0, first_pos + starts - window + 1)
            steps = -(-(k_end - k_begin) // 32)
            total += int(steps.sum()) + 8 * len(steps)
            longest = max(longest, int(steps.max()))
        path, work = -(-longest // halves) * cost.trip_us, total * heads * cost.step_ns * 1e-3
        return cost.start_us + (path ** 4 + work ** 4) ** 0.25
    ways = [(per, halves) for halves in sorted({1, max(1, int(most_halves))}) for per in sorted({min(4, most), most})]
    return min(ways, key=lambda way: (estimate(*way), way[1], way[0]))


WORKGROUP_RANGES = 4    # key ranges of a tile that one workgroup (four wavefronts) walks and merges itself


def _single_token_plan(row_ctx: np.ndarray, window: Optional[int], splits: int, merge_in_workgroup: int = 0) -> AttentionPlan:
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
    start = (k_begin // KEY_ALIGN) * KEY_ALIGN
    per = -(-(k_end - start) // (ranges if merge_in_workgroup else splits))
    per = -(-per // KEY_ALIGN) * KEY_ALIGN
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
                         tuning: AttentionTuning = DEFAULT_TUNING, tile_halves: int = 1, tile_min_workgroups: int = 0) -> AttentionPlan:
    """Cut the step's rows into tiles of tokens and, where that pays, ranges of keys.

    With ``fixed_splits`` every tile gets exactly that many items (some may be empty), so the
    arrays have the same shape whatever the contexts are.  With ``workgroup_tiles`` (the number of tiles a
    workgroup of that kernel takes, which the kernel library tells) rows with many tiles (portions of prompts) go
    to the kernel in which the tiles of a workgroup share the keys they load; ``tile_halves`` says whether that kernel
    can split a workgroup's keys between two halves of its wavefronts (2) or not (1), ``tile_min_workgroups`` how many
    workgroups a launch of it needs to be worth while (a kernel whose steps are slow is bounded by its longest
    workgroup unless there are many)."""
    _, tokens_per_tile, group_tiles = group_tiling(group_size)
    row_len = np.asarray(row_len, dtype=np.int64)
    row_ctx = np.asarray(row_ctx, dtype=np.int64)
    merge_in_workgroup = WORKGROUP_RANGES if merge_in_workgroup is True else int(merge_in_workgroup)
    if merge_in_workgroup and not (len(row_len) and int(row_len.min()) == 1 == int(row_len.max())):
        raise ValueError("key ranges are merged in the workgroup only in steps of one token per row")
    if merge_in_workgroup not in (0, 2, WORKGROUP_RANGES) or (merge_in_workgroup == 2 and len(row_len) % 2):
        raise ValueError("a workgroup merges four key ranges of one tile, or two ranges of each of two tiles (an even number of rows)")
    if (merge_in_workgroup or (single_token_shortcut and fixed_splits is not None)) and len(row_len) \
            and int(row_len.min()) == 1 == int(row_len.max()):
        return _single_token_plan(row_ctx, window, int(fixed_splits or merge_in_workgroup or 1), merge_in_workgroup)
    tiles_per_row = -(-row_len // tokens_per_tile)
    waves_unsplit = int(tiles_per_row.sum()) * n_kv_heads * group_tiles
    items, slots, merges, tiles = [], [], [], []
    n_slots = 0
    per_workgroup, halves = 0, 1
    if workgroup_tiles and fixed_splits is None:
        chosen = _workgroup_tiles_that_pay(row_len, row_ctx, tiles_per_row, tokens_per_tile, n_kv_heads * group_tiles, window,
                                           int(workgroup_tiles), tuning, int(tile_halves))
        per_workgroup, halves = chosen if isinstance(chosen, tuple) else (chosen, 1)
        if per_workgroup and tile_min_workgroups:
            groups = sum(-(-int(n) // (per_workgroup * tokens_per_tile)) for n, tiles_of_row in zip(row_len, tiles_per_row)
                         if tiles_of_row >= MIN_TILES_FOR_WORKGROUPS)
            if groups * n_kv_heads * group_tiles < tile_min_workgroups:
                per_workgroup, halves = 0, 1
    for row in range(len(row_len)):
        n, ctx = int(row_len[row]), int(row_ctx[row])
        first_pos = ctx - n
        if per_workgroup and tiles_per_row[row] >= MIN_TILES_FOR_WORKGROUPS:
            span = per_workgroup * tokens_per_tile
            for q0 in range(0, n, span):
                k_begin = 0 if window is None else max(0, first_pos + q0 - window + 1)
                tiles.append((row, q0, k_begin, first_pos + min(q0 + span, n)))
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
                splits = min(MAX_SPLITS, max(1, target_waves // max(1, waves_unsplit)), max(1, n_keys // MIN_KEYS_PER_SPLIT))
            if splits <= 1:
                items.append((row, q0, k_begin, k_end))
                slots.append(-1)
                continue
            start = (k_begin // KEY_ALIGN) * KEY_ALIGN
            per = -(-(k_end - start) // splits)
            per = -(-per // KEY_ALIGN) * KEY_ALIGN        # at most `splits` items, each a multiple of KEY_ALIGN keys
            first_slot = n_slots
            count = 0
            while start < k_end or (fixed_splits is not None and count < splits):
                lo, hi = max(start, k_begin), min(start + per, k_end)
                items.append((row, q0, lo, max(lo, hi)) if lo < k_end else (row, q0, k_end, k_end))
                slots.append(n_slots)
                n_slots += 1
                count += 1
                start += per
            merges.append((row, q0, first_slot, count))
    items = np.asarray(items, dtype=np.int32).reshape(-1, 4)
    merges = np.asarray(merges, dtype=np.int32).reshape(-1, 4)
    tiles.sort(key=lambda tile: tile[2] - tile[3])       # most keys first: the long tiles must not start last
    tiles = np.asarray(tiles, dtype=np.int32).reshape(-1, 4)
    return AttentionPlan(items, np.asarray(slots, dtype=np.int32), merges, n_slots, tiles, per_workgroup if len(tiles) else 0,
                         halves if len(tiles) else 1)


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

    def prepare(self, ctx):
        key = self.plan_key()
        if ctx.has_plan(key):
            return
        fixed = None
        tuning = tuning_of(ctx.ops, DEFAULT_TUNING)
        if ctx.static_max_keys is not None:          # a step whose shapes must not depend on the contexts
            fixed = fixed_split_count(ctx.n_rows, self.group_size, self.n_kv_heads, ctx.static_max_keys, tuning.target_waves)
        # Where a workgroup can merge a tile's key ranges itself, the merge launch and the partial results go:
        #  * short contexts (the step says so, and keeps saying so for as long as its shape is replayed): four ranges a tile;
        #  * so many rows that a tile gets four ranges anyway;
        #  * two ranges a tile: two tiles to a workgroup, if the rows come in pairs.  (Two or three ranges in a workgroup
        #    of one tile leave wavefronts idle through the others' walk: a tenth slower at 64 rows behind 4,096 tokens.)
        in_workgroup = 0
        if ctx.n_tokens == ctx.n_rows:
            if ctx.short_contexts:
                in_workgroup = fixed = WORKGROUP_RANGES
            elif fixed == WORKGROUP_RANGES or (fixed == 2 and ctx.n_rows % 2 == 0):
                in_workgroup = fixed
        per_workgroup = ctx.ops.attention_workgroup_tiles(ctx.dtype, self.head_dim, ctx.page_size)
        halves = ctx.ops.attention_tile_halves(ctx.dtype, self.head_dim) if per_workgroup else 1
        fewest = ctx.ops.attention_tile_min_workgroups(ctx.dtype) if per_workgroup else 0
        plan = build_attention_plan(ctx.h_row_len, ctx.h_row_ctx, self.group_size, self.n_kv_heads, self.window,
                                    target_waves=tuning.target_waves, fixed_splits=fixed, workgroup_tiles=per_workgroup,
                                    merge_in_workgroup=in_workgroup, tuning=tuning, tile_halves=halves, tile_min_workgroups=fewest)
        ctx.set_plan(key, {
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
