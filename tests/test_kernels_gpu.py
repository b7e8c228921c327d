"""Each HIP kernel alone against its plain torch twin, at other sizes than the engine's tests use:
head sizes in steps of 16, groups that are no power of two, widths and vocabularies that are no
power of two, page sizes from 4 to 500.  Inputs are built so that faults show: a far key that must
win, a window's edge, pages in scrambled order, a page used again."""
import math

import numpy as np
import pytest
import torch

from llmserver_amd.parts.attention import build_attention_plan, group_tiling
from torch_ops import TorchOps

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = {torch.float32: dict(atol=2e-5, rtol=1e-5), torch.bfloat16: dict(atol=2e-2, rtol=2e-2)}


@pytest.fixture(scope="module")
def ops():
    """The kernels themselves are under test here: the table that sends some shapes to the library instead of a
    few-row kernel, which serving consults, is switched off (it has a test of its own below)."""
    from llmserver_amd.kernels import default_ops
    ops = default_ops()
    ops.consult_choices = False
    yield ops
    ops.consult_choices = True


class Ctx:
    def empty(self, shape, dtype=None):
        return torch.empty(shape, device=DEV, dtype=dtype)


def close(a, b, dtype):
    torch.testing.assert_close(a.float(), b.float(), **TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [8, 100, 1000, 4104, 9001])
def test_add_rmsnorm(ops, dtype, width):
    print(f"add_rmsnorm {dtype} width {width}", flush=True)
    torch.manual_seed(width)
    x = (3 * torch.randn(11, width, device=DEV)).to(dtype)
    delta = torch.randn(11, width, device=DEV).to(dtype)
    weight = 1 + 0.2 * torch.randn(width, device=DEV)
    for d in (delta, None):
        got_x, ref_x = x.clone(), x.clone()
        got, ref = torch.empty_like(x), torch.empty_like(x)
        ops.add_rmsnorm(got_x, d, weight, 1e-5, got)
        TorchOps().add_rmsnorm(ref_x, d, weight, 1e-5, ref)
        assert torch.equal(got_x, ref_x)                          # the residual sum is rounded once, identically
        close(got, ref, dtype)
    rows = torch.tensor([10, 0, 3, 3], device=DEV, dtype=torch.int32)
    got_x = x.clone()
    got, ref = (torch.empty(4, width, device=DEV, dtype=dtype) for _ in range(2))
    ops.add_rmsnorm(got_x, delta, weight, 1e-5, got, rows)
    TorchOps().add_rmsnorm(x.clone(), delta, weight, 1e-5, ref, rows)
    assert torch.equal(got_x, x)                                  # selected rows only: the stream is left alone
    close(got, ref, dtype)


def test_rmsnorm_sums_in_32_bit(ops):
    """Ten thousand bfloat16 ones: a 16-bit running sum would stall at 256."""
    x = torch.ones(1, 10000, device=DEV, dtype=torch.bfloat16)
    out = torch.empty_like(x)
    ops.add_rmsnorm(x, None, torch.ones(10000, device=DEV), 0.0, out)
    assert torch.equal(out, x)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("inter", [4, 100, 6152, 13001])
def test_swiglu_embedding_bias(ops, dtype, inter):
    print(f"swiglu/embedding/bias {dtype} {inter}", flush=True)
    torch.manual_seed(inter)
    gate_up = (4 * torch.randn(7, 2 * inter, device=DEV)).to(dtype)
    got, ref = (torch.empty(7, inter, device=DEV, dtype=dtype) for _ in range(2))
    ops.swiglu(gate_up, got)
    TorchOps().swiglu(gate_up, ref)
    close(got, ref, dtype)
    table = torch.randn(301, inter, device=DEV).to(dtype)
    ids = torch.tensor([300, 0, 17, 17, 299], device=DEV, dtype=torch.int32)
    out = torch.empty(5, inter, device=DEV, dtype=dtype)
    ops.embedding(table, ids, out)
    assert torch.equal(out, table[ids.long()])
    y = torch.randn(7, inter, device=DEV).to(dtype)
    bias = torch.randn(inter, device=DEV)
    ref = (y.float() + bias).to(dtype)
    ops.add_bias_(y, bias)
    assert torch.equal(y, ref)


def make_cache(n_pages, n_kv, page, d, dtype):
    keys = torch.zeros(n_pages, n_kv, page, d, device=DEV, dtype=dtype)
    values = torch.zeros(n_pages, n_kv, d, page, device=DEV, dtype=dtype)
    return keys, values


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n_q, n_kv, d, page", [(4, 2, 16, 16), (6, 2, 48, 12), (8, 8, 64, 4), (5, 1, 80, 8), (32, 8, 128, 16), (2, 1, 256, 500)])
def test_qk_norm_rope_kv_write(ops, dtype, n_q, n_kv, d, page):
    print(f"qk_norm_rope_kv_write {dtype} {n_q}/{n_kv} d{d} page{page}", flush=True)
    torch.manual_seed(d + n_q)
    # portions and decoded tokens; with a long portion the values take the tiled path, at starts that are and are no multiple of four
    lens, starts = ([5, 1, 23], [0, 700, 37]) if d not in (64, 128) else ([300, 1, 23], [401, 1, 37]) if d == 128 else ([130, 200, 2], [64, 7, 3])
    rows = len(lens)
    n_pages = 200 if page < 500 else 8
    width = max(-(-(s + n) // page) for s, n in zip(starts, lens))
    table = torch.full((rows, width), -1, dtype=torch.int32)
    n_pages = max(n_pages, sum(-(-(s + n) // page) for s, n in zip(starts, lens)) + 2)
    perm = torch.randperm(n_pages)
    used = 0
    for r, (s, n) in enumerate(zip(starts, lens)):
        blocks = -(-(s + n) // page)
        table[r, :blocks] = perm[used:used + blocks].int()
        used += blocks
    positions = torch.cat([torch.arange(s, s + n) for s, n in zip(starts, lens)]).int()
    token_row = torch.cat([torch.full((n,), r) for r, n in enumerate(lens)]).int()
    tokens = len(positions)
    qkv = torch.randn(tokens, (n_q + 2 * n_kv) * d, device=DEV).to(dtype)
    qw, kw = 1 + 0.2 * torch.randn(d, device=DEV), 1 + 0.2 * torch.randn(d, device=DEV)
    inv_freq = (1.0 / (1e6 ** (torch.arange(0, d, 2).float() / d))).to(DEV)
    table, positions, token_row = table.to(DEV), positions.to(DEV), token_row.to(DEV)
    cos_sin = ops.rotary_table(positions, inv_freq)
    torch.testing.assert_close(cos_sin, TorchOps().rotary_table(positions, inv_freq), atol=2e-6, rtol=0)
    for norm, rope, write in ((True, True, True), (False, True, True), (True, False, True), (True, True, False)):
        got_qkv, ref_qkv = qkv.clone(), qkv.clone()
        got_k, got_v = make_cache(n_pages, n_kv, page, d, dtype)
        ref_k, ref_v = make_cache(n_pages, n_kv, page, d, dtype)
        args = (table, token_row, positions, qw if norm else None, kw if norm else None, 1e-6, cos_sin if rope else None, page, n_q, n_kv, d, write)
        ops.qk_norm_rope_kv_write(got_qkv, got_k, got_v, *args)
        TorchOps().qk_norm_rope_kv_write(ref_qkv, ref_k, ref_v, *args)
        close(got_qkv[:, :n_q * d], ref_qkv[:, :n_q * d], dtype)
        close(got_k, ref_k, dtype)
        assert torch.equal(got_v, ref_v)
        if not write:
            assert not got_k.any() and not got_v.any()


def attention_case(ops, dtype, n_q, n_kv, d, page, lens, ctxs, window=None, needle=True, seed=0, target_waves=None, workgroup_tiles=None,
                   merge_in_workgroup=False, tile_halves=1, tile_walk=None):
    """Random q/k/v through both implementations.  Pages are handed out in scrambled order from a
    pool that first held other data (as if used before).  With ``needle``, one far key per request
    is made to dominate its first query's softmax."""
    torch.manual_seed(seed)
    rows = len(lens)
    n_pages = sum(-(-c // page) for c in ctxs) + 3
    keys = (5 * torch.randn(n_pages, n_kv, page, d, device=DEV)).to(dtype)      # stale data of earlier users
    values = (5 * torch.randn(n_pages, n_kv, d, page, device=DEV)).to(dtype)
    perm = torch.randperm(n_pages)
    width = max(-(-c // page) for c in ctxs)
    table = torch.full((rows, width), -1, dtype=torch.int32)
    used = 0
    tokens = sum(lens)
    qkv = torch.randn(tokens, (n_q + 2 * n_kv) * d, device=DEV).to(dtype)
    row_start = np.cumsum([0] + list(lens[:-1])).astype(np.int32)
    for r, c in enumerate(ctxs):
        blocks = -(-c // page)
        first = 0 if window is None else max(0, c - lens[r] - window + 1) // page
        table[r, :blocks] = perm[used:used + blocks].int()
        used += blocks
        k = torch.randn(c, n_kv, d, device=DEV)
        v = torch.randn(c, n_kv, d, device=DEV)
        if needle and c > 40:
            far = 3 if window is None else max(0, c - lens[r] - window + 1)       # the oldest key the first query may see
            q0 = qkv[row_start[r], :d].float()
            k[far, 0] = 6.0 * q0 / q0.norm() * math.sqrt(d) / max(1.0, float(q0.norm()) / math.sqrt(d))
            v[far, 0] = 10.0
        place = torch.arange(c)
        pages = table[r].long()[place // page].to(DEV)
        keys[pages, :, (place % page).to(DEV), :] = k.to(dtype)
        values[pages, :, :, (place % page).to(DEV)] = v.to(dtype)
        table[r, :first] = -1                                                     # pages a window has passed are gone
    # workgroup_tiles: None lets the plan choose between the tile counts the kernel offers, 0 keeps every row out of the
    # prompt-portion kernel, 4 or 8 fixes the count (and ``tile_halves`` and ``tile_walk``, the most steps of 32 keys a
    # workgroup is left with, the rest going to workgroups of their own).
    from llmserver_amd.parts import attention as attention_module
    most = ops.attention_workgroup_tiles(dtype, d, page) if workgroup_tiles is None or workgroup_tiles else 0
    chooser = attention_module._workgroup_tiles_that_pay
    most_halves = ops.attention_tile_halves(dtype, d) if most else 1
    key_ranges = ops.attention_tile_key_ranges(dtype, d) if most else 1
    if workgroup_tiles:
        assert workgroup_tiles <= most and tile_halves <= most_halves and (tile_walk is None or key_ranges > 1)
        attention_module._workgroup_tiles_that_pay = lambda *args, **kwargs: (workgroup_tiles, tile_halves, tile_walk)
    try:
        plan = build_attention_plan(lens, ctxs, n_q // n_kv, n_kv, window, workgroup_tiles=0 if merge_in_workgroup else most,
                                    merge_in_workgroup=merge_in_workgroup, tile_halves=most_halves, tuning=ops.attention_tuning,
                                    tile_key_ranges=key_ranges, **({} if target_waves is None else {"target_waves": target_waves}))
    finally:
        attention_module._workgroup_tiles_that_pay = chooser
    staged = {"items": torch.from_numpy(plan.items).to(DEV), "item_slot": torch.from_numpy(plan.item_slot).to(DEV),
              "merges": torch.from_numpy(plan.merges).to(DEV), "tiles": torch.from_numpy(plan.tiles).to(DEV), "n_tiles": len(plan.tiles),
              "n_items": len(plan.items), "n_merges": len(plan.merges), "n_slots": plan.n_slots, "tiles_per_workgroup": plan.tiles_per_workgroup,
              "tile_halves": plan.tile_halves, "merge_in_workgroup": int(plan.merge_in_workgroup),
              "most_splits": int(plan.merges[:, 3].max()) if len(plan.merges) else 0}
    if plan.tile_slots is not None:
        staged["tile_slots"] = torch.from_numpy(plan.tile_slots).to(DEV)
    t = lambda a: torch.tensor(a, dtype=torch.int32, device=DEV)
    got = torch.zeros(tokens, n_q * d, device=DEV, dtype=dtype)
    ref = torch.zeros_like(got)
    table = table.to(DEV)
    scale = d ** -0.5
    ops.paged_attention(qkv, got, keys, values, table, t(row_start), t(lens), t(ctxs), staged, scale, window, page, n_q, n_kv, d, Ctx())
    TorchOps().paged_attention(qkv, ref, keys, values, table.clamp(min=0), t(row_start), t(lens), t(ctxs), None, scale, window, page, n_q, n_kv, d, None)
    torch.cuda.synchronize()
    assert torch.isfinite(got.float()).all()
    close(got, ref, dtype)
    return plan, ref


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n_q, n_kv, d, page", [(4, 2, 16, 16), (8, 2, 32, 8), (6, 2, 48, 12), (3, 3, 64, 4), (32, 8, 128, 16),
                                                (5, 1, 80, 20), (20, 1, 16, 16), (16, 1, 112, 64), (2, 1, 256, 500), (7, 7, 96, 32)])
def test_attention_mixed_batch(ops, dtype, n_q, n_kv, d, page):
    """Decoded tokens at contexts straddling pages and key steps beside portions of prompts with and without a prefix."""
    print(f"attention mixed {dtype} {n_q}/{n_kv} d{d} page{page}", flush=True)
    lens = [1, 1, 1, 17, 40, 2, 1]
    ctxs = [1, 33, 300, 17, 140, 65, 1025]
    plan, _ = attention_case(ops, dtype, n_q, n_kv, d, page, lens, ctxs, seed=n_q * d)
    assert plan.n_slots > 0                                     # long contexts of single tokens were split


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n_q, n_kv, d, page", [(4, 2, 16, 16), (6, 2, 48, 12), (32, 8, 128, 16), (5, 1, 80, 8), (20, 1, 64, 16), (2, 1, 256, 64)])
@pytest.mark.parametrize("window", [None, 40])
@pytest.mark.parametrize("per_tile", [4, 2])
def test_attention_key_ranges_merged_in_the_workgroup(ops, dtype, n_q, n_kv, d, page, window, per_tile):
    """Steps of single tokens whose tiles get four key ranges each, walked by the four wavefronts of one workgroup and
    merged there (no partial results, no merge launch): contexts of one token (three ranges empty), at the edges of
    pages and key steps, with a far key that decides the first query; queries and keys prepared by the separate kernel."""
    print(f"attention merged in the workgroup {dtype} {n_q}/{n_kv} d{d} page{page} window {window}, {per_tile} ranges a tile", flush=True)
    ctxs = [1, 2, 3, 4, 5, 31, 32, 33, 63, 64, 65, 127, 128, 129, 300, 511, 512, 1025]
    plan, ref = attention_case(ops, dtype, n_q, n_kv, d, page, [1] * len(ctxs), ctxs, window=window, seed=n_q * d + 1, merge_in_workgroup=per_tile)
    assert plan.merge_in_workgroup == per_tile and len(plan.items) == per_tile * len(ctxs) and plan.n_slots == 0 and len(plan.merges) == 0
    if window is None:
        assert float(ref[-1, :d].float().mean()) > 5.0           # the far key won the last row's first head
    if per_tile == 2:
        with pytest.raises(ValueError):                          # a row of two tokens: tiles in pairs are for single tokens only
            build_attention_plan([1, 2], [5, 9], n_q // n_kv, n_kv, window, merge_in_workgroup=per_tile)
        return
    # Rows of several tokens (portions of prompts, as captured steps of short contexts have them): every tile of every row
    # gets four ranges, some of them empty, and the workgroup merges them; portions with and without a prefix, tiles that
    # are not full, a row of one token among them.
    lens = [17, 1, 40, 2, 128, 5]
    ctxs = [17, 33, 140, 65, 512, 300]
    plan, _ = attention_case(ops, dtype, n_q, n_kv, d, page, lens, ctxs, window=window, seed=n_q * d + 2, merge_in_workgroup=per_tile)
    assert plan.merge_in_workgroup == 4 and len(plan.items) % 4 == 0 and plan.n_slots == 0 and len(plan.merges) == 0
    assert (plan.item_slot == -1).all() and len(plan.tiles) == 0


@pytest.mark.parametrize("n_q, n_kv, d, page", [(32, 8, 128, 16), (4, 2, 64, 8), (20, 1, 64, 16), (6, 3, 192, 12), (2, 1, 256, 64)])
@pytest.mark.parametrize("window", [None, 40])
def test_attention_decode_fusion(ops, n_q, n_kv, d, page, window):
    """A step of single tokens with the q/k norm, the rotation and the cache write left to the attention kernel,
    against the two separate kernels and against the plain twin: outputs and what lands in the cache; with and
    without norm and rotation; reading a cache that another layer has written; with key ranges split evenly as
    captured steps do (trailing ranges are then empty and must not count the new token twice)."""
    print(f"attention decode fusion {n_q}/{n_kv} d{d} page{page} window {window}", flush=True)
    dtype = torch.bfloat16
    torch.manual_seed(n_q + d)
    ctxs = [1, 2, 33, 300, 1025, 64, 65]
    rows = len(ctxs)
    lens = [1] * rows
    n_pages = sum(-(-c // page) for c in ctxs) + 3
    keys0 = (5 * torch.randn(n_pages, n_kv, page, d, device=DEV)).to(dtype)
    values0 = (5 * torch.randn(n_pages, n_kv, d, page, device=DEV)).to(dtype)
    perm = torch.randperm(n_pages)
    width = max(-(-c // page) for c in ctxs)
    table = torch.full((rows, width), -1, dtype=torch.int32)
    used = 0
    for r, c in enumerate(ctxs):
        blocks = -(-c // page)
        table[r, :blocks] = perm[used:used + blocks].int()
        used += blocks
        place = torch.arange(c - 1)
        pages = table[r].long()[place // page].to(DEV)
        keys0[pages, :, (place % page).to(DEV), :] = torch.randn(c - 1, n_kv, d, device=DEV).to(dtype)
        values0[pages, :, :, (place % page).to(DEV)] = torch.randn(c - 1, n_kv, d, device=DEV).to(dtype)
        first = 0 if window is None else max(0, c - window) // page
        table[r, :first] = -1
    table = table.to(DEV)
    t = lambda a: torch.tensor(a, dtype=torch.int32, device=DEV)
    row_start, row_len, row_ctx = t(list(range(rows))), t(lens), t(ctxs)
    positions, token_row = t([c - 1 for c in ctxs]), t(list(range(rows)))
    qkv = torch.randn(rows, (n_q + 2 * n_kv) * d, device=DEV).to(dtype)
    qw, kw = 1 + 0.2 * torch.randn(d, device=DEV), 1 + 0.2 * torch.randn(d, device=DEV)
    inv_freq = (1.0 / (1e6 ** (torch.arange(0, d, 2).float() / d))).to(DEV)
    cos_sin = ops.rotary_table(positions, inv_freq)
    scale = d ** -0.5
    for fixed in (None, 8, "in the workgroup"):
        in_workgroup = fixed == "in the workgroup"                           # four key ranges a tile, merged by the workgroup that walks them
        plan = build_attention_plan(lens, ctxs, n_q // n_kv, n_kv, window, fixed_splits=8 if in_workgroup else fixed,
                                    merge_in_workgroup=4 if in_workgroup else 0)
        staged = {"items": torch.from_numpy(plan.items).to(DEV), "item_slot": torch.from_numpy(plan.item_slot).to(DEV),
                  "merges": torch.from_numpy(plan.merges).to(DEV), "n_items": len(plan.items), "n_merges": len(plan.merges),
                  "n_slots": plan.n_slots, "merge_in_workgroup": int(plan.merge_in_workgroup)}
        assert plan.n_slots > 0 or window is not None or in_workgroup        # long contexts are split, unless a window keeps them short
        assert not in_workgroup or (len(plan.items) == 4 * rows and plan.n_slots == 0 and not len(plan.merges))
        for norm, rope in ((True, True),) if in_workgroup else ((True, True), (False, True), (True, False)):
            w_q, w_k, cs = (qw if norm else None), (kw if norm else None), (cos_sin if rope else None)
            # the separate kernels, and the plain twin of both
            sep_qkv, sep_k, sep_v = qkv.clone(), keys0.clone(), values0.clone()
            ops.qk_norm_rope_kv_write(sep_qkv, sep_k, sep_v, table.clamp(min=0), token_row, positions, w_q, w_k, 1e-6, cs, page, n_q, n_kv, d, True)
            sep_out = torch.zeros(rows, n_q * d, device=DEV, dtype=dtype)
            ops.paged_attention(sep_qkv, sep_out, sep_k, sep_v, table, row_start, row_len, row_ctx, staged, scale, window, page, n_q, n_kv, d, Ctx())
            ref_qkv, ref_k, ref_v = qkv.clone(), keys0.clone(), values0.clone()
            TorchOps().qk_norm_rope_kv_write(ref_qkv, ref_k, ref_v, table.clamp(min=0), token_row, positions, w_q, w_k, 1e-6, cs, page, n_q, n_kv, d, True)
            ref_out = torch.zeros_like(sep_out)
            TorchOps().paged_attention(ref_qkv, ref_out, ref_k, ref_v, table.clamp(min=0), row_start, row_len, row_ctx, None, scale, window, page, n_q, n_kv, d, None)
            # fused, writing the cache
            raw, got_k, got_v = qkv.clone(), keys0.clone(), values0.clone()
            got = torch.zeros_like(sep_out)
            ops.paged_attention(raw, got, got_k, got_v, table, row_start, row_len, row_ctx, staged, scale, window, page, n_q, n_kv, d, Ctx(),
                                decode_fusion=(w_q, w_k, 1e-6, cs, True))
            torch.cuda.synchronize()
            assert torch.equal(raw, qkv)                                     # the projection is read, not rewritten
            close(got, ref_out, dtype)
            torch.testing.assert_close(got.float(), sep_out.float(), atol=2e-2, rtol=2e-2)
            close(got_k, ref_k, dtype)
            assert torch.equal(got_v, ref_v)
            # fused, reading a cache that already holds the new token (another layer wrote it)
            kept_k, kept_v = sep_k.clone(), sep_v.clone()
            got = torch.zeros_like(sep_out)
            ops.paged_attention(raw, got, kept_k, kept_v, table, row_start, row_len, row_ctx, staged, scale, window, page, n_q, n_kv, d, Ctx(),
                                decode_fusion=(w_q, w_k, 1e-6, cs, False))
            close(got, ref_out, dtype)
            assert torch.equal(kept_k, sep_k) and torch.equal(kept_v, sep_v)
    with pytest.raises(ValueError):                                          # a row with two tokens
        ops.paged_attention(torch.zeros(rows + 1, (n_q + 2 * n_kv) * d, device=DEV, dtype=dtype), torch.zeros(rows + 1, n_q * d, device=DEV, dtype=dtype),
                            keys0, values0, table, row_start, row_len, row_ctx, staged, scale, window, page, n_q, n_kv, d, Ctx(),
                            decode_fusion=(qw, kw, 1e-6, cos_sin, True))
    assert not ops.decode_fusion_fits(torch.float32, d) and not ops.decode_fusion_fits(dtype, 80)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_long_context_splits_and_needle(ops, dtype):
    print(f"attention long {dtype}", flush=True)
    plan, ref = attention_case(ops, dtype, 8, 2, 128, 16, [1, 3], [2049, 1500], seed=3)
    assert len(plan.merges) == 2 and plan.n_slots >= 4           # both rows were cut into several key ranges
    assert float(ref[0, :128].float().mean()) > 5.0             # the far key won: its value (10) dominates the first head
    attention_case(ops, dtype, 8, 2, 128, 16, [1, 3], [2049, 1500], seed=3, target_waves=1)      # same, unsplit
    attention_case(ops, dtype, 4, 4, 64, 16, [600], [600], seed=4, target_waves=10 ** 6)         # a whole prompt, split to the limit
    plan, ref = attention_case(ops, dtype, 4, 1, 64, 16, [1], [16384], seed=5)                   # one token behind 16,383: 128 key ranges
    assert int(plan.merges[:, 3].max()) == 128 and float(ref[0, :64].float().mean()) > 5.0
    plan, _ = attention_case(ops, dtype, 4, 1, 64, 16, [1], [8300], seed=6)                      # 87 ranges: more than one wavefront has lanes
    assert 64 < int(plan.merges[:, 3].max()) < 128


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [1, 7, 16, 33, 100])
def test_attention_window_edge(ops, dtype, window):
    """The oldest key inside the window carries the needle; the one before it must not be read (its page is gone)."""
    print(f"attention window {window} {dtype}", flush=True)
    attention_case(ops, dtype, 4, 2, 32, 8, [1, 1, 25, 60, 2], [50, 300, 125, 60, 200], window=window, seed=window)
    attention_case(ops, dtype, 4, 2, 32, 8, [1, 9], [700, 400], window=window, seed=window, target_waves=10 ** 6)


@pytest.mark.parametrize("n_q, n_kv, d, page", [(4, 2, 16, 16), (8, 2, 32, 8), (6, 2, 48, 24), (32, 8, 128, 16), (5, 1, 80, 40), (20, 1, 16, 8),
                                                (2, 1, 256, 504), (16, 16, 64, 64), (12, 4, 96, 32), (3, 1, 112, 48)])
@pytest.mark.parametrize("window", [None, 40])
def test_attention_prompt_portions_in_workgroup_tiles(ops, n_q, n_kv, d, page, window):
    """Long portions of prompts, with and without a prefix, beside decoded tokens: the portions go
    through the kernel whose four wavefronts share the keys they load (bfloat16), with one tile of 16 pairs per
    wavefront and with two.  Pages of 16 keys or a multiple (a wavefront's quarter of a step lies in one page) and
    other multiples of 8 (every lane looks its page up)."""
    print(f"attention workgroup tiles {n_q}/{n_kv} d{d} page{page} window {window}", flush=True)
    lens = [333, 1, 200, 97, 1]
    ctxs = [333, 90, 777, 130, 400]
    plan, _ = attention_case(ops, torch.bfloat16, n_q, n_kv, d, page, lens, ctxs, window=window, seed=n_q + d)
    assert len(plan.tiles) > 0 and len(plan.items) > 0
    attention_case(ops, torch.bfloat16, n_q, n_kv, d, page, lens, ctxs, window=window, seed=n_q + d, workgroup_tiles=0)
    for per_workgroup in (4, 8):                                   # one and two tiles per wavefront
        for halves in (1, 2):                                      # the keys of a workgroup whole, or in two halves of its wavefronts
            if per_workgroup <= ops.attention_workgroup_tiles(torch.bfloat16, d) and halves <= ops.attention_tile_halves(torch.bfloat16, d):
                plan, _ = attention_case(ops, torch.bfloat16, n_q, n_kv, d, page, lens, ctxs, window=window, seed=n_q + d,
                                         workgroup_tiles=per_workgroup, tile_halves=halves)
                assert (plan.tiles_per_workgroup, plan.tile_halves) == (per_workgroup, halves) and len(plan.tiles) > 0


@pytest.mark.parametrize("n_q, n_kv, d, page", [(32, 8, 128, 16), (4, 2, 16, 16), (8, 2, 32, 8), (6, 2, 48, 24), (5, 1, 80, 40), (20, 1, 64, 16),
                                                (2, 1, 256, 64), (12, 4, 96, 32), (3, 1, 112, 48)])
@pytest.mark.parametrize("window", [None, 300])
def test_attention_key_ranges_of_workgroup_tiles(ops, n_q, n_kv, d, page, window):
    """Rows of few tokens behind long contexts in the prompt-portion kernel, their keys cut into ranges for workgroups
    of their own and the partial results merged: with four and with eight tiles to a workgroup, keys whole or in halves,
    ranges of 2, 5 and 16 steps; beside decoded tokens, whole prompts and rows too short for that kernel; a far key
    decides the first query of every row, so a range that is lost or counted twice shows."""
    print(f"attention key ranges of workgroup tiles {n_q}/{n_kv} d{d} page{page} window {window}", flush=True)
    lens = [70, 1, 9, 333, 2, 37, 130]
    ctxs = [1500, 400, 777, 333, 65, 1061, 2200]
    dtype = torch.bfloat16
    assert ops.attention_tile_key_ranges(dtype, d) == 128 and ops.attention_tile_key_ranges(torch.float32, d) == 1
    plan, _ = attention_case(ops, dtype, n_q, n_kv, d, page, lens, ctxs, window=window, seed=n_q + d)      # as the plan chooses
    assert len(plan.tiles) > 0 and len(plan.items) > 0
    for per_workgroup in (4, 8):
        for halves in (1, 2):
            if per_workgroup > ops.attention_workgroup_tiles(dtype, d) or halves > ops.attention_tile_halves(dtype, d):
                continue
            for walk in (2, 5, 16):
                plan, _ = attention_case(ops, dtype, n_q, n_kv, d, page, lens, ctxs, window=window, seed=n_q + d,
                                         workgroup_tiles=per_workgroup, tile_halves=halves, tile_walk=walk)
                if window is not None and walk == 16:                        # a window of 300 keys is 11 steps at most
                    assert plan.tile_slots is None
                    continue
                assert plan.tile_slots is not None and (plan.tile_slots[:, 0] >= 0).any() and plan.n_slots > 0
                assert window is not None or int(plan.merges[:, 3].max()) >= min(128, 2200 // (32 * walk))
                assert (plan.tile_slots[:, 0] < 0).any() or walk < 5         # the whole prompt's first tiles have few keys


def test_pages_the_workgroup_kernel_does_not_take_go_to_wavefronts_of_their_own(ops):
    """The bfloat16 prompt-portion kernel fetches 8 keys of a value row at a time: with pages of 4, 12 or 20 keys the
    plan keeps every row out of it (the kernel library says so), and a plan that does not is refused."""
    for page in (4, 12, 20):
        assert ops.attention_workgroup_tiles(torch.bfloat16, 32, page) == 0
        plan, _ = attention_case(ops, torch.bfloat16, 8, 2, 32, page, [333, 1, 97], [333, 90, 130], seed=page)
        assert len(plan.tiles) == 0 and len(plan.items) > 0
    assert ops.attention_workgroup_tiles(torch.bfloat16, 32, 8) > 0 and ops.attention_workgroup_tiles(torch.float32, 32, 12) == 4
    from llmserver_amd.parts.attention import build_attention_plan
    plan = build_attention_plan([333], [333], 4, 2, None, workgroup_tiles=4)
    staged = {"items": torch.zeros((0, 4), dtype=torch.int32, device=DEV), "item_slot": torch.zeros((0,), dtype=torch.int32, device=DEV),
              "merges": torch.zeros((0, 4), dtype=torch.int32, device=DEV), "tiles": torch.from_numpy(plan.tiles).to(DEV), "n_tiles": len(plan.tiles),
              "n_items": 0, "n_merges": 0, "n_slots": 0, "tiles_per_workgroup": 4, "tile_halves": 1}
    qkv = torch.zeros(333, (8 + 2 * 2) * 32, device=DEV, dtype=torch.bfloat16)
    out = torch.zeros(333, 8 * 32, device=DEV, dtype=torch.bfloat16)
    keys = torch.zeros(30, 2, 12, 32, device=DEV, dtype=torch.bfloat16)
    values = torch.zeros(30, 2, 32, 12, device=DEV, dtype=torch.bfloat16)
    t = lambda a: torch.tensor(a, dtype=torch.int32, device=DEV)
    with pytest.raises(ValueError, match="does not take pages of 12 keys"):
        ops.paged_attention(qkv, out, keys, values, torch.zeros((1, 28), dtype=torch.int32, device=DEV), t([0]), t([333]), t([333]), staged,
                            32 ** -0.5, None, 12, 8, 2, 32, Ctx())


@pytest.mark.parametrize("n_q, n_kv, d, page", [(4, 2, 16, 16), (8, 2, 32, 8), (6, 2, 48, 12), (32, 8, 128, 16), (5, 1, 80, 20), (2, 1, 256, 500)])
@pytest.mark.parametrize("window", [None, 40])
def test_attention_prompt_portions_in_workgroup_tiles_float32(ops, n_q, n_kv, d, page, window):
    """The float32 form of the prompt-portion kernel (four tiles to a workgroup, true 32-bit products) against the twin
    at float32 tolerances, with a needle among the far keys, beside decoded tokens and short portions."""
    print(f"attention workgroup tiles float32 {n_q}/{n_kv} d{d} page{page} window {window}", flush=True)
    assert ops.attention_workgroup_tiles(torch.float32, d) == 4 and ops.attention_tile_halves(torch.float32, d) == 1
    lens = [333, 1, 200, 97, 1]
    ctxs = [333, 90, 777, 130, 400]
    plan, _ = attention_case(ops, torch.float32, n_q, n_kv, d, page, lens, ctxs, window=window, seed=n_q + d, workgroup_tiles=4)
    assert len(plan.tiles) > 0 and len(plan.items) > 0 and plan.tiles_per_workgroup == 4


def test_attention_refuses_sizes_it_cannot_take(ops):
    from llmserver_amd.kernels import build
    with pytest.raises(ValueError, match="head sizes"):
        build.attention_module(True, 24)
    with pytest.raises(ValueError, match="head sizes"):
        build.attention_module(True, 272)
    qkv = torch.zeros(1, 4 * 16, device=DEV)
    out = torch.zeros(1, 2 * 16, device=DEV)
    keys, values = torch.zeros(2, 1, 6, 16, device=DEV), torch.zeros(2, 1, 16, 6, device=DEV)
    one = torch.ones(1, dtype=torch.int32, device=DEV)
    plan = {"items": torch.zeros(1, 4, dtype=torch.int32, device=DEV), "item_slot": -one, "merges": torch.zeros(0, 4, dtype=torch.int32, device=DEV),
            "n_items": 1, "n_merges": 0, "n_slots": 0, "n_tiles": 0}
    with pytest.raises(ValueError, match="multiple of 4"):
        ops.paged_attention(qkv, out, keys, values, torch.zeros(1, 1, dtype=torch.int32, device=DEV), 0 * one, one, one, plan, 1.0, None, 6, 2, 1, 16, Ctx())
    with pytest.raises(TypeError):
        ops.swiglu(torch.zeros(1, 4, device=DEV, dtype=torch.float16), torch.zeros(1, 2, device=DEV, dtype=torch.float16))
    with pytest.raises(ValueError, match="GPU"):
        ops.swiglu(torch.zeros(1, 4), torch.zeros(1, 2))


@pytest.mark.parametrize("vocab", [7, 301, 1024, 151936])
def test_sampling(ops, vocab):
    print(f"sampling vocab {vocab}", flush=True)
    torch.manual_seed(vocab)
    rows = 9
    logits = (3 * torch.randn(rows, vocab, device=DEV)).float()
    logits[0, vocab // 2] = logits[0, vocab - 1] = 50.0                         # a tie: the first maximum wins
    temperature = torch.tensor([0.0, 0.0, 0.8, 0.8, 1.0, 2.5, 0.3, 0.8, 0.8], device=DEV)
    uniform = torch.tensor([0.5, 0.1, 0.0, 0.999999, 0.5, 0.25, 0.75, 0.5, 0.123], device=DEV)
    out = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
    ops.sample(logits, temperature, uniform, out)
    got = out.tolist()
    assert got[0] == vocab // 2 and got[1] == int(torch.argmax(logits[1]))
    for row in range(2, rows):
        weights = torch.exp((logits[row].double() - logits[row].double().max()) / float(temperature[row]))
        cdf = torch.cumsum(weights, 0) / weights.sum()
        u, index = float(uniform[row]), got[row]
        low = float(cdf[index - 1]) if index else 0.0
        assert 0 <= index < vocab and low - 1e-4 <= u <= float(cdf[index]) + 1e-4, (row, index, low, u, float(cdf[index]))
    # frequencies follow the distribution
    few = torch.tensor([[0.0, 1.0, 2.0, -1.0, 0.5]], device=DEV).repeat(4000, 1)
    draws = torch.empty(4000, dtype=torch.int32, device=DEV)
    ops.sample(few, torch.full((4000,), 0.7, device=DEV), torch.rand(4000, device=DEV), draws)
    freq = torch.bincount(draws.long().cpu(), minlength=5).double() / 4000
    expected = torch.softmax(few[0].double().cpu() / 0.7, 0)
    assert float((freq - expected).abs().max()) < 0.03


@pytest.mark.parametrize("rows", [1, 3, 8, 16, 17, 33, 64])
@pytest.mark.parametrize("n, k", [(16, 8), (100, 72), (301, 4096), (6144, 1000), (4096, 12288), (200, 5120), (77, 1536),
                                  (130, 1792)])
def test_skinny_gemm(ops, rows, n, k):
    """The weight-streaming product against a float64 product of the same bfloat16 values: widths and
    output sizes that are no multiple of the tiles, widths that give a wavefront 4, 5, 6, 7 or 8 k steps
    at a time, whole and partly used tiles of the weight per workgroup, one or two of them, float32 and
    bfloat16 results."""
    print(f"skinny gemm rows {rows} n {n} k {k}", flush=True)
    torch.manual_seed(rows * n + k)
    x = torch.randn(rows, k, device=DEV).to(torch.bfloat16)
    w = (torch.randn(n, k, device=DEV) / k ** 0.5).to(torch.bfloat16)
    expected = (x.double() @ w.double().t()).float()
    saved = ops.skinny_rows
    try:
        ops.skinny_rows = 64
        for per in (0, 16, 8, 3, 24, 32, 17) if rows <= 16 else (0, 16, 12):
            got32 = ops.linear(x, w, out_float32=True, rows_per_workgroup=per)
            got16 = ops.linear(x, w, rows_per_workgroup=per)
            assert got32.dtype == torch.float32 and got16.dtype == torch.bfloat16
            torch.testing.assert_close(got32, expected, atol=2e-4, rtol=1e-4)          # 32-bit accumulation of exact products
            torch.testing.assert_close(got16.float(), expected, atol=2e-2, rtol=1e-2)
    finally:
        ops.skinny_rows = saved
    with pytest.raises(RuntimeError):
        ops._gemm_refusal_check = ops._gemm.lsa_gemm_skinny(0, x.data_ptr(), w.data_ptr(), got16.data_ptr(), 65, n, k, 0, None, 0, 0.0, None, None)
        if ops._gemm_refusal_check != 0:
            raise RuntimeError("refused")


@pytest.mark.parametrize("rows", [1, 7, 16, 17, 33, 64, 65, 300])
@pytest.mark.parametrize("n, k", [(48, 72), (301, 520), (1030, 264), (96, 33), (6144, 4096)])
def test_product_with_bias_is_rounded_once(ops, rows, n, k):
    """``x w^T + b`` in bfloat16: the bias joins the float32 sums and the result is rounded once, so it lies within
    half a bfloat16 step of the exact value (a product that is rounded before the bias is added misses by up to a
    whole step, and by more where the bias cancels the product).  Through the few-row kernels and the library."""
    print(f"product with bias rows {rows} n {n} k {k}", flush=True)
    torch.manual_seed(rows + n + k)
    x = torch.randn(rows, k, device=DEV).to(torch.bfloat16)
    w = (torch.randn(n, k, device=DEV) / k ** 0.5).to(torch.bfloat16)
    bias = torch.randn(n, device=DEV).to(torch.bfloat16).float()
    exact = x.double() @ w.double().t() + bias.double()
    got = ops.linear(x, w, bias=bias, bias_rounded=bias.to(torch.bfloat16))
    assert got.dtype == torch.bfloat16 and got.shape == (rows, n)
    half_step = exact.abs() * 2.0 ** -8
    float32_sums = 1e-6 * (x.double().abs() @ w.double().abs().t() + bias.double().abs())
    assert bool(((got.double() - exact).abs() <= half_step + float32_sums).all())
    # a bias that bfloat16 does not hold is added to the rounded product (and so is every bias in float32)
    odd_bias = bias + 2.0 ** -12
    got = ops.linear(x, w, bias=odd_bias, bias_rounded=None)
    torch.testing.assert_close(got.float(), (exact + 2.0 ** -12).float(), atol=3e-2, rtol=2e-2)
    got = ops.linear(x.float(), w.float(), bias=odd_bias)
    torch.testing.assert_close(got, (exact + 2.0 ** -12).float(), atol=2e-4, rtol=1e-4)


@pytest.mark.parametrize("rows", [9, 16, 17, 32, 33, 48, 49, 64, 65, 96, 97, 128])
@pytest.mark.parametrize("n, k", [(48, 72), (301, 4096), (4096, 12288), (2050, 1000), (200, 5128), (8192, 64), (5120, 520), (127, 264),
                                  (10880, 3840), (8192, 4104)])
def test_product_in_partial_sums(ops, rows, n, k):
    """The product for 17 to 128 rows, which leaves partial sums over ranges of the inner dimension, against a float64
    product of the same bfloat16 values: one range and many, ranges that end inside a staged slab, sizes that are no
    multiple of the tiles; ranges of six, five (an odd number) and four slabs and a last range of one whole slab and a
    ragged one, which beyond 64 rows go through the form that asks for the weights a slab ahead.  Then the kernel that adds them up, adds the result to a residual stream and normalises,
    against its twin."""
    print(f"product in partial sums rows {rows} n {n} k {k}", flush=True)
    torch.manual_seed(rows * n + k)
    x = torch.randn(rows, k, device=DEV).to(torch.bfloat16)
    w = (torch.randn(n, k, device=DEV) / k ** 0.5).to(torch.bfloat16)
    expected = (x.double() @ w.double().t()).float()
    parts = ops._gemm.lsa_gemm_split_parts(rows, n, k)
    assert parts >= 1
    sums = torch.full((parts, rows, n), float("nan"), device=DEV)                          # every element must be written
    assert ops._gemm.lsa_gemm_split(x.data_ptr(), w.data_ptr(), sums.data_ptr(), rows, n, k, None) == 0
    torch.testing.assert_close(sums.sum(0), expected, atol=2e-4, rtol=1e-4)
    offered = ops.linear_partial_sums(x, w, few_rows_too=True)
    assert (offered is None) == (parts < 2)                                               # nothing to split: left to the library
    if offered is not None:
        assert torch.equal(offered, sums)
    for refused in (0, 129):
        assert ops._gemm.lsa_gemm_split_parts(refused, n, k) == -1
    assert ops._gemm.lsa_gemm_split_parts(rows, n, k + 4) == -1
    resid = (2 * torch.randn(rows, n, device=DEV)).to(torch.bfloat16)
    weight = 1 + 0.2 * torch.randn(n, device=DEV)
    got_x, ref_x = resid.clone(), resid.clone()
    got, ref = torch.empty_like(resid), torch.empty_like(resid)
    ops.add_rmsnorm(got_x, sums, weight, 1e-5, got)
    TorchOps().add_rmsnorm(ref_x, sums, weight, 1e-5, ref)
    # the parts are added up in another order than the twin's: a sum on a rounding boundary may differ by one step
    assert float((got_x.float() - ref_x.float()).abs().gt(0).float().mean()) < 0.01
    torch.testing.assert_close(got_x.float(), ref_x.float(), atol=4e-2, rtol=1e-2)
    close(got, ref, torch.bfloat16)
    picked = torch.tensor([rows - 1, 0, 3, 3], device=DEV, dtype=torch.int32)
    got_x = resid.clone()
    got, ref = (torch.empty(4, n, device=DEV, dtype=torch.bfloat16) for _ in range(2))
    ops.add_rmsnorm(got_x, sums, weight, 1e-5, got, picked)
    TorchOps().add_rmsnorm(resid.clone(), sums, weight, 1e-5, ref, picked)
    assert torch.equal(got_x, resid)
    close(got, ref, torch.bfloat16)


@pytest.mark.parametrize("rows", [1, 5, 8, 9, 16])
@pytest.mark.parametrize("n, k", [(48, 72), (301, 4096), (4096, 12288), (6144, 1000), (200, 5120), (8192, 64), (5120, 512), (2048, 256)])
def test_skinny_gemm_with_row_scale_and_stream_update(ops, rows, n, k):
    """The few-row product with a norm folded in on either side, against the separate kernels' twins:
    as a consumer it reads the stream times the norm's weights and divides its rows by the stream's rms,
    which it gets as partial sums of squares; as a producer it adds its result to a residual stream and
    writes what the next product needs of the norm that follows."""
    print(f"row scale and stream update rows {rows} n {n} k {k}", flush=True)
    torch.manual_seed(rows + n + k)
    w = (torch.randn(n, k, device=DEV) / k ** 0.5).to(torch.bfloat16)
    stream = (3 * torch.randn(rows, k, device=DEV)).to(torch.bfloat16)
    norm_weight = 1 + 0.2 * torch.randn(k, device=DEV)
    eps = 1e-5
    # consumer: partial sums over an arbitrary split of the rows (here 7 uneven parts)
    bounds = [0, 1, k // 5, k // 3, k // 2, k - 3, k - 1, k]
    squares = stream.float() ** 2
    square_sums = torch.stack([squares[:, a:b].sum(1) for a, b in zip(bounds, bounds[1:])], dim=1).contiguous()
    weighted = (stream.float() * norm_weight).to(torch.bfloat16)
    rstd = torch.rsqrt(squares.double().sum(1, keepdim=True) / k + eps)
    expected = (weighted.double() @ w.double().t()) * rstd
    for per in (0, 16, 12, 24, 32):
        for out32 in (False, True):
            got = ops.linear_few_rows(weighted, w, out_float32=out32, rows_per_workgroup=per, row_scale=(square_sums, eps))
            assert got.dtype == (torch.float32 if out32 else torch.bfloat16)
            torch.testing.assert_close(got.double(), expected, atol=2e-4 if out32 else 3e-2, rtol=1e-4 if out32 else 2e-2)
    # ... and it is the product of the normalised stream, up to the rounding of the normalised values
    normed = torch.empty_like(stream)
    TorchOps().add_rmsnorm(stream.clone(), None, norm_weight, eps, normed)
    torch.testing.assert_close(expected, normed.double() @ w.double().t(), atol=3e-2, rtol=3e-2)
    # producer: y added to a residual stream of width n, the next norm's weights applied, squares summed per 16 columns
    x = torch.randn(rows, k, device=DEV).to(torch.bfloat16)
    resid = (2 * torch.randn(rows, n, device=DEV)).to(torch.bfloat16)
    next_weight = 1 + 0.2 * torch.randn(n, device=DEV)
    y = (x.double() @ w.double().t()).float().to(torch.bfloat16)
    want_stream = (resid.float() + y.float()).to(torch.bfloat16)
    want_weighted = (want_stream.float() * next_weight).to(torch.bfloat16)
    for per in (0, 16, 12, 24, 32):
        kept = resid.clone()
        got_stream, got_weighted, got_sums = ops.linear_into_stream(x, w, kept, next_weight, rows_per_workgroup=per)
        assert torch.equal(kept, resid)
        # y is rounded once to bfloat16 before the sum, as the separate kernels do; a product that lands on a
        # rounding boundary may differ by one step of bfloat16
        torch.testing.assert_close(got_stream.float(), want_stream.float(), atol=4e-2, rtol=1e-2)
        assert float((got_stream.float() - want_stream.float()).abs().gt(0).float().mean()) < 0.02
        torch.testing.assert_close(got_weighted.float(), (got_stream.float() * next_weight).to(torch.bfloat16).float(), atol=0, rtol=0)
        assert got_sums.shape[0] == rows and (per == 0 or got_sums.shape[1] == -(-n // per))
        torch.testing.assert_close(got_sums.sum(1), (got_stream.float() ** 2).sum(1), atol=1e-3, rtol=1e-5)
    # chained: the producer's outputs feed a consumer of width n
    w2 = (torch.randn(72, n, device=DEV) / n ** 0.5).to(torch.bfloat16)
    got_stream, got_weighted, got_sums = ops.linear_into_stream(weighted, w, resid, next_weight, row_scale=(square_sums, eps))
    if n % 8:
        assert ops.linear_few_rows(got_weighted, w2, row_scale=(got_sums, eps)) is None          # widths in steps of 8 only
    elif got_sums.shape[1] <= (ops.SCALE_PARTS if rows <= 8 else ops.SCALE_PARTS // 2):
        chained = ops.linear_few_rows(got_weighted, w2, out_float32=True, row_scale=(got_sums, eps))
        normed = torch.empty_like(got_stream)
        TorchOps().add_rmsnorm(got_stream.clone(), None, next_weight, eps, normed)
        torch.testing.assert_close(chained.double(), normed.double() @ w2.double().t(), atol=3e-2, rtol=3e-2)
    else:
        assert ops.linear_few_rows(got_weighted, w2, row_scale=(got_sums, eps)) is None
    # more rows than the fused epilogues take
    many = torch.zeros(17, k, device=DEV, dtype=torch.bfloat16)
    saved = ops.skinny_rows
    try:
        ops.skinny_rows = 64
        assert ops.linear_into_stream(many, w, torch.zeros(17, n, device=DEV, dtype=torch.bfloat16), next_weight) is None
        assert ops.linear_few_rows(many, w, row_scale=(torch.ones(17, 4, device=DEV), eps)) is None
    finally:
        ops.skinny_rows = saved


@pytest.mark.parametrize("rows", [1, 5, 8, 13, 16])
@pytest.mark.parametrize("inter, k", [(8, 16), (104, 72), (12288, 4096), (1000, 1000), (264, 5120), (40, 1536), (72, 1792)])
def test_gated_product_with_activation_in_the_epilogue(ops, rows, inter, k):
    print(f"gated product rows {rows} inter {inter} k {k}", flush=True)
    torch.manual_seed(rows + inter + k)
    x = torch.randn(rows, k, device=DEV).to(torch.bfloat16)
    w = (torch.randn(2 * inter, k, device=DEV) / k ** 0.5).to(torch.bfloat16)
    gate_up = x.double() @ w.double().t()
    expected = (torch.nn.functional.silu(gate_up[:, :inter]) * gate_up[:, inter:]).float()
    square_sums = torch.rand(rows, 5, device=DEV) * k
    rstd = torch.rsqrt(square_sums.double().sum(1, keepdim=True) / k + 1e-6)
    scaled = (torch.nn.functional.silu(gate_up[:, :inter] * rstd) * gate_up[:, inter:] * rstd).float()
    for per in (0, -1, 16, 12, 5):
        got = ops.linear_gated(x, w, pairs_per_workgroup=per)
        assert got.shape == (rows, inter) and got.dtype == torch.bfloat16
        torch.testing.assert_close(got.float(), expected, atol=2e-2, rtol=2e-2)
        got = ops.linear_gated(x, w, pairs_per_workgroup=per, row_scale=(square_sums, 1e-6))
        torch.testing.assert_close(got.float(), scaled, atol=2e-2, rtol=2e-2)
    assert ops.linear_gated(torch.zeros(17, k, device=DEV, dtype=torch.bfloat16), w, row_scale=(torch.ones(17, 4, device=DEV), 1e-6)) is None


@pytest.mark.parametrize("rows", [17, 24, 32, 33])
@pytest.mark.parametrize("inter, k", [(12288, 4096), (9000, 264), (10001, 72), (16384, 1000), (20000, 1000), (8192, 512), (1000, 1000)])
def test_gated_product_beyond_few_rows(ops, rows, inter, k):
    """17 to 32 rows: the product that shares the activations through LDS, with the activation in its epilogue, where
    the weight has rows enough for one workgroup to take the whole inner dimension; elsewhere it is not offered."""
    print(f"gated product beyond few rows {rows} inter {inter} k {k}", flush=True)
    torch.manual_seed(rows + inter + k)
    x = torch.randn(rows, k, device=DEV).to(torch.bfloat16)
    w = (torch.randn(2 * inter, k, device=DEV) / k ** 0.5).to(torch.bfloat16)
    got = ops.linear_gated(x, w)
    offered = bool(ops._gemm.lsa_gemm_split_gated_fits(rows, inter, k))
    assert offered == (rows <= 32 and inter > 8192)               # tiles of 64 pairs: more than half as many as compute units
    assert (got is not None) == offered
    if got is not None:
        gate_up = x.double() @ w.double().t()
        expected = (torch.nn.functional.silu(gate_up[:, :inter]) * gate_up[:, inter:]).float()
        assert got.shape == (rows, inter) and got.dtype == torch.bfloat16
        torch.testing.assert_close(got.float(), expected, atol=2e-2, rtol=2e-2)
    assert ops.linear_gated(torch.zeros(49, k, device=DEV, dtype=torch.bfloat16), w) is None
    assert ops._gemm.lsa_gemm_split_gated(x.data_ptr(), w.data_ptr(), x.data_ptr(), 16, inter, k, None) == -1


def test_library_product_in_ranges_of_the_inner_dimension_by_table(ops):
    """A product of a few hundred rows whose result joins the residual stream goes through the library whole, or as a
    batched product of two or four ranges of the inner dimension with float32 results, as the table of choices says;
    unknown shapes go whole and nothing is timed unless the caller is inside ``measuring()``.  Either way the sums that
    reach the stream are right."""
    from llmserver_amd.kernels.choices import ChoiceTable, choice_key
    print("library product in ranges by table", flush=True)
    torch.manual_seed(9)
    rows, out, width = 200, 320, 1536
    x = torch.randn(rows, width, device=DEV).to(torch.bfloat16)
    w = (torch.randn(out, width, device=DEV) / width ** 0.5).to(torch.bfloat16)
    expected = (x.double() @ w.double().t()).float()
    keys = {parts: choice_key(f"parts{parts}", 256, out, width, False, False) for parts in (2, 4)}
    bucket = type(ops)._parts_bucket
    assert bucket(129) == 192 and bucket(256) == 256 and bucket(257) == 384 and bucket(1024) == 1024
    saved_table, ops.choices = ops.choices, ChoiceTable(ops.choices.device_name)
    ops.consult_choices = True
    try:
        assert ops.library_parts(x, w) == 0 and ops.linear_partial_sums(x, w) is None and not ops.choices.entries
        for best in (2, 4, 0):
            for parts, key in keys.items():
                ops.choices.entries[key] = parts == best
            assert ops.library_parts(x, w) == best
            sums = ops.linear_partial_sums(x, w)
            if not best:
                assert sums is None
                continue
            assert sums.shape == (best, rows, out) and sums.dtype == torch.float32
            torch.testing.assert_close(sums.sum(0), expected, atol=2e-3, rtol=2e-3)
            stream = torch.randn(rows, out, device=DEV).to(torch.bfloat16)
            before = stream.float()
            normed = torch.empty_like(stream)
            ops.add_rmsnorm(stream, sums, torch.ones(out, device=DEV), 1e-6, normed)
            torch.testing.assert_close(stream.float(), (before + expected).to(torch.bfloat16).float(), atol=2e-2, rtol=1e-2)
        assert ops.library_parts(x[:, :1532].contiguous(), w[:, :1532].contiguous()) == 0       # ranges must be multiples of 8
        assert ops.library_parts(x[:100], w) == 0 and ops.library_parts(torch.zeros(1100, width, device=DEV, dtype=torch.bfloat16), w) == 0
        ops.choices = ChoiceTable(ops.choices.device_name)
        with ops.measuring():
            chosen = ops.library_parts(x, w)
        assert chosen in (0, 2, 4) and set(ops.choices.measured) == set(keys.values())
        assert [ops.choices.entries[keys[parts]] for parts in (2, 4)] == [chosen == 2, chosen == 4]
        assert ops.library_parts(x, w) == chosen and ops._flush is None
    finally:
        ops.choices = saved_table
        ops.consult_choices = False


def test_few_row_kernel_or_library_by_table(ops, tmp_path):
    """A shape goes the way the table of choices says; a shape the table does not know goes the few-row kernel's way
    and nothing is timed, unless the caller is inside ``measuring()``: then it is timed once, entered into the table
    and can be saved.  Either way the product is right.  While a graph is recorded nothing is timed."""
    from llmserver_amd.kernels.choices import ChoiceTable, choice_key
    print("few-row kernel or library by table", flush=True)
    torch.manual_seed(5)
    x = torch.randn(8, 512, device=DEV).to(torch.bfloat16)
    w = (torch.randn(1024, 512, device=DEV) / 512 ** 0.5).to(torch.bfloat16)
    expected = (x.double() @ w.double().t()).float()
    plain_key, gated_key = choice_key("plain", 8, 1024, 512, False, False), choice_key("gated", 8, 1024, 512, False, False)
    saved_table, ops.choices = ops.choices, ChoiceTable(ops.choices.device_name)
    ops.consult_choices = True
    try:
        for _ in range(2):
            torch.testing.assert_close(ops.linear(x, w).float(), expected, atol=2e-2, rtol=1e-2)
        assert not ops.choices.entries and ops._flush is None      # an unknown shape: no timing, no entry
        with ops.measuring():
            for _ in range(2):
                torch.testing.assert_close(ops.linear(x, w).float(), expected, atol=2e-2, rtol=1e-2)
        assert list(ops.choices.entries) == [plain_key] == list(ops.choices.measured)
        assert ops._flush is None                                    # the buffer that empties the caches is given back
        path = str(tmp_path / "choices.json")
        assert ops.choices.save(path) == 1
        again = ChoiceTable.load(ops.choices.device_name, [path])
        assert again.entries == ops.choices.entries and ChoiceTable.load("another GPU", [path]).entries == {}
        for forced in (True, False):
            ops.choices.entries[plain_key] = forced
            torch.testing.assert_close(ops.linear(x, w).float(), expected, atol=2e-2, rtol=1e-2)
        ops.choices.entries[gated_key] = True
        assert ops.linear_gated(x, w) is None and ops.linear_gated(x, w, pairs_per_workgroup=8) is not None
        ops.choices.entries[gated_key] = False
        assert ops.linear_gated(x, w) is not None
        ops.choices = ChoiceTable(ops.choices.device_name)
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            ops.linear(x, w)                              # (warm-up on the side stream, as graph capture wants it)
        torch.cuda.current_stream().wait_stream(side)
        with ops.measuring():
            with torch.cuda.graph(graph):
                captured = ops.linear(x, w)
        assert not ops.choices.entries                    # nothing was measured during the capture
        graph.replay()
        torch.cuda.synchronize()
        torch.testing.assert_close(captured.float(), expected, atol=2e-2, rtol=1e-2)
    finally:
        ops.choices = saved_table
        ops.consult_choices = False


def test_plain_read_runs_and_refuses_what_it_cannot_split():
    """The bandwidth tool's kernel: any number of workgroups and threads it is documented for, nothing read past the end."""
    from llmserver_amd.kernels import bandwidth, library
    lib = library.load("elementwise")
    data = torch.ones(1 << 16, device=DEV)
    sink = torch.zeros(1, device=DEV)
    for workgroups, threads in ((1, 64), (7, 256), (256, 1024)):
        assert lib.lsa_plain_read(data.data_ptr(), sink.data_ptr(), data.numel() * 4, workgroups, threads, None) == 0
    assert lib.lsa_plain_read(data.data_ptr(), sink.data_ptr(), data.numel() * 4, 4, 100, None) == -1
    assert lib.lsa_plain_read(data.data_ptr(), sink.data_ptr(), 16, 4, 256, None) == -1
    torch.cuda.synchronize()
    assert float(sink) == 0.0
    assert 0 < bandwidth.measure(8, 64, 256, repeats=1) < 1.0
