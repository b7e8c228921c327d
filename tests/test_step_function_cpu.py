"""The step function, the cache and the replay driver on the CPU (with the torch twins of the
kernels): every way of cutting and batching gives the plain implementation's logits."""
import io

import numpy as np
import pytest
import torch

import traces
from helpers import model_folder, plain_logits, random_tokens
from llmserver_amd.engine.replay import make_runner, replay
from tiny_configs import CASES
from torch_ops import TorchOps


def requests_for(case, lengths, seed0=100):
    vocab = CASES[case][0]["vocab_size"]
    return {f"q{i}": random_tokens(vocab, n, seed0 + i) for i, n in enumerate(lengths)}, {f"q{i}": (n, seed0 + i) for i, n in enumerate(lengths)}


def run(case, steps, max_tokens, tmp_path, page_size=None, fused=False):
    page = page_size or CASES[case][2]
    runner = make_runner(model_folder(case), "float32", max_tokens, page, device="cpu", ops=TorchOps(fused=fused))
    report = io.StringIO()
    replay(runner, traces.to_lines(steps).splitlines(), str(tmp_path), report)
    assert report.getvalue().split() == [w for s in steps for w in ("done", str(s["step"]))]
    runner.cache.check_invariants()
    assert not runner.cache.requests and min(runner.cache.available_pages()) == runner.cache.groups[0].pool.num_pages
    return traces.collect(steps, str(tmp_path), CASES[case][0]["vocab_size"]), runner


def check(case, results, meta, atol=3e-5):
    for (rid, position), logits in results.items():
        n, seed = meta[rid]
        expected = plain_logits(case, n, seed)[position].numpy()
        np.testing.assert_allclose(logits, expected, atol=atol, rtol=1e-4, err_msg=f"{rid} position {position}")
    assert len(results) == sum(n for n, _ in meta.values())


@pytest.mark.parametrize("case", ["A", "B", "C"])
@pytest.mark.parametrize("schedule", ["whole", "tail", "portions", "mixed"])
def test_every_schedule_matches_the_plain_implementation(case, schedule, tmp_path):
    lengths = (5, 17, 33, 70, 100, 41, 64, 1, 90, 130, 20, 77) if schedule == "mixed" else (70, 33, 100)
    requests, meta = requests_for(case, lengths)
    if schedule == "whole":
        steps = traces.whole(requests)
    elif schedule == "tail":
        steps = traces.tail_decoded(requests, 32)
    elif schedule == "portions":
        steps = traces.changing_portions(requests)
    else:
        steps = traces.mixed(requests, seed=7, budget_tokens=256)
        assert max(len(s["entries"]) for s in steps) >= 3
        assert any(len(e["tokens"]) == 1 for s in steps for e in s["entries"]) and any(len(e["tokens"]) > 8 for s in steps for e in s["entries"])
    budget = traces.peak_tokens(steps)
    results, runner = run(case, steps, budget, tmp_path)
    if schedule == "mixed":
        assert sum(lengths) > 2 * budget            # more tokens ran through than the pool holds: pages were used again
    check(case, results, meta)


@pytest.mark.parametrize("case", ["A", "B", "C"])
@pytest.mark.parametrize("schedule", ["tail", "mixed"])
def test_the_fused_dataflow_matches_the_plain_implementation(case, schedule, tmp_path):
    """The same with the twins of the fused kernels offered to the parts: projections that add their result to the
    residual stream and prepare the next norm, projections that apply a prepared norm as a scale of their rows, and
    single-token steps whose attention normalises, rotates and stores the new token itself."""
    lengths = (5, 17, 33, 70, 100, 41, 64, 1, 90, 130, 20, 77) if schedule == "mixed" else (70, 33, 100)
    requests, meta = requests_for(case, lengths)
    steps = traces.tail_decoded(requests, 32) if schedule == "tail" else traces.mixed(requests, seed=7, budget_tokens=256)
    results, runner = run(case, steps, traces.peak_tokens(steps), tmp_path, fused=True)
    check(case, results, meta)
    calls = runner.ops.fused_calls
    assert calls["into_stream"] > 0 and calls["row_scale"] > 0 and calls["gated"] > 0
    assert calls["partial_sums"] > 0
    if schedule == "tail":
        assert calls["decode_attention"] > 0


def test_a_step_refuses_what_does_not_fit(tmp_path):
    runner = make_runner(model_folder("A"), "float32", 64, 16, device="cpu", ops=TorchOps())
    from llmserver_amd.cache import CacheExhaustedError
    from llmserver_amd.engine import StepEntry
    runner.cache.open("a")
    with pytest.raises(ValueError, match="vocabulary"):
        runner.step([StepEntry("a", [5, 999], [0])])
    with pytest.raises(ValueError, match="wanted place"):
        runner.step([StepEntry("a", [5, 6], [2])])
    with pytest.raises(ValueError, match="twice"):
        runner.step([StepEntry("a", [5], []), StepEntry("a", [6], [])])
    with pytest.raises(ValueError, match="no tokens"):
        runner.step([StepEntry("a", [], [])])
    with pytest.raises(KeyError):
        runner.step([StepEntry("nobody", [5], [])])
    with pytest.raises(CacheExhaustedError):
        runner.step([StepEntry("a", [1] * 65, [])])
    assert runner.cache.record("a").num_computed == 0 and runner.cache.available_pages() == [4]
    out = runner.step([StepEntry("a", [1, 2, 3], [])])
    assert out.shape == (0, 256) and runner.cache.record("a").num_computed == 3


def test_filler_rows_of_a_captured_shape(tmp_path):
    """Decoding steps are filled up to one of a few numbers of rows; the rows added are first tokens of nobody's, each
    on a scratch page of its own behind the pool, and the requests' own rows and pages are what they were."""
    from llmserver_amd.engine import StepEntry
    from llmserver_amd.engine.step import padded_rows
    sizes = [padded_rows(rows) for rows in range(1, 200)]
    assert all(rows <= size < rows + 16 and size <= max(rows + 1, rows * 5 // 4) for rows, size in zip(range(1, 200), sizes))
    assert sizes == sorted(sizes) and len(set(sizes[:64])) == 18 and all(padded_rows(size) == size for size in sizes)
    runner = make_runner(model_folder("A"), "float32", 256, 16, device="cpu", ops=TorchOps())
    for name, n in (("a", 5), ("b", 20)):
        runner.cache.open(name)
        runner.step([StepEntry(name, list(range(1, n + 1)), [])])
    entries = [StepEntry("a", [7], [0]), StepEntry("b", [9], [0])]
    plain = runner.build_context(entries)
    filled = runner.build_context(entries, filler_rows=3)
    pool_pages = runner.cache.groups[0].pool.num_pages
    assert filled.n_rows == 5 and filled.n_tokens == 5 and filled.n_out == 5
    assert list(filled.h_row_ctx) == [6, 21, 1, 1, 1] and list(filled.h_row_len) == [1] * 5
    table = filled.h_tables[0]
    assert (table[:2, :plain.h_tables[0].shape[1]] == plain.h_tables[0]).all()
    scratch = runner.cache.groups[0].scratch_pages          # (rows of one token take the last of the scratch pages)
    assert list(table[2:, 0]) == [pool_pages + scratch - 1, pool_pages + scratch - 2, pool_pages + scratch - 3] and (table[2:, 1:] == -1).all()
    assert runner.cache.groups[0].keys.shape[1] == pool_pages + scratch and scratch >= 16 + 512 // 16
    runner.cache.check_invariants()


def test_a_step_with_portions_filled_up_to_a_captured_shape():
    """A small step that brings a portion of a prompt beside a decoded token is filled up to fixed numbers of rows and
    tokens: rows of one token of nobody's, and one more row of nobody's with the tokens that are missing, the start of
    a prompt on the first scratch pages (or no tokens at all, if the numbers fit).  The requests' own rows come out
    as without the fillers, the attention plan has the shape that any rows of these numbers would give, and the
    wanted places are every row's last token."""
    import numpy as np
    from llmserver_amd.engine import StepEntry
    runner = make_runner(model_folder("A"), "float32", 256, 16, device="cpu", ops=TorchOps())
    tokens = {"a": list(range(1, 41)), "b": list(range(50, 63))}
    for name in tokens:
        runner.cache.open(name)
    runner.step([StepEntry("a", tokens["a"][:20], [])])
    runner.step([StepEntry("b", tokens["b"][:12], [])])
    entries = [StepEntry("a", tokens["a"][20:31], [10]), StepEntry("b", tokens["b"][12:], [0])]        # 11 + 1 tokens
    plain = runner.build_context(entries)
    shapes = []
    for filler_tokens in (19, 0):                     # filled up to 32 tokens (with one filler row of one token); or the numbers fit
        filled = runner.build_context(entries, table_width=64, filler_rows=1, filler_tokens=filler_tokens, want_last=True)
        assert filled.n_rows == 4 and filled.n_tokens == 13 + filler_tokens and filled.n_out == 4
        assert list(filled.h_row_len) == [11, 1, 1, filler_tokens] and list(filled.h_row_ctx) == [31, 13, 1, filler_tokens]
        assert list(filled.h_logit_idx[:3]) == [10, 11, 12] and 0 <= filled.h_logit_idx[3] < filled.n_tokens
        assert list(filled.h_token_ids[:12]) == list(plain.h_token_ids) and list(filled.h_positions[13:]) == list(range(filler_tokens))
        table, pool_pages = filled.h_tables[0], runner.cache.groups[0].pool.num_pages
        assert (table[:2, :plain.h_tables[0].shape[1]] == plain.h_tables[0]).all()
        assert list(table[3, :2]) == ([pool_pages, pool_pages + 1] if filler_tokens else [-1, -1])
        filled.static_max_keys = 64 * 16
        runner.model.prepare(filled)
        plan = filled.get_plan(runner.model.blocks[0].mixer.plan_key())
        shapes.append((plan["items"].shape, plan["merges"].shape, plan["n_slots"], plan["n_tiles"]))
        # every token of every row meets its keys: the tiles of a row cover its tokens, each tile's ranges its keys
        covered = {}
        for row, q0, k_begin, k_end in plan["items"].tolist():
            covered.setdefault((row, q0), set()).update(range(k_begin, k_end))
        for row, (length, context) in enumerate(zip(filled.h_row_len, filled.h_row_ctx)):
            for q0 in range(0, int(length), 8):       # (two query heads to a KV head: eight tokens to a tile)
                assert covered[(row, q0)] == set(range(int(context) - int(length) + min(q0 + 8, int(length)))), (row, q0)
    # (the second has 19 tokens fewer: its shape is that of a smaller captured number of tokens, but rows and ranges agree)
    assert shapes[0][0][0] == (32 // 8 + 4) * (shapes[0][0][0] // (32 // 8 + 4)) and shapes[0][3] == 0 and shapes[1][3] == 0
    runner.cache.check_invariants()


def test_which_steps_with_portions_are_captured():
    """The shape a small step with portions is filled up to, and the steps that stay eager: too many rows or tokens,
    logits wanted elsewhere than at a row's end, a shape met for the first time, and steps that the GPU bounds anyway
    (estimated from the model's own sizes, so every run decides alike)."""
    from llmserver_amd.engine import StepEntry
    from llmserver_amd.engine.step import PORTION_ROWS, PORTION_TOKENS, padded_tokens
    assert [padded_tokens(n) for n in (1, 8, 9, 100, 512, 513)] == [8, 8, 16, 128, 512, None] and list(PORTION_TOKENS) == sorted(PORTION_TOKENS)
    runner = make_runner(model_folder("A"), "float32", 2048, 16, device="cpu", ops=TorchOps())
    runner.use_graphs = True                      # (only the keys are asked for here; nothing is captured on the CPU)
    for name in ("a", "b", "c"):
        runner.cache.open(name)
    runner.cache.advance("a", 0)
    step = [StepEntry("a", list(range(40)), [39]), StepEntry("b", [5], [0])]
    assert runner._graph_key(step) is None        # met for the first time
    key = runner._graph_key(step)
    assert key == ("portions", 3, 48, 64, 3, ("short contexts",))      # two rows and one of fillers; 41 tokens filled up to 48; all rows' ends wanted
    assert runner._graph_key([StepEntry("a", list(range(44)), [43]), StepEntry("c", [1, 2, 3], [2])]) == key       # other lengths, the same shape
    assert runner._graph_key([StepEntry("a", list(range(40)), []), StepEntry("b", [5, 6], [])]) is None            # nothing wanted: another shape, first meeting
    assert runner._graph_key([StepEntry("a", list(range(40)), []), StepEntry("b", [5, 6], [])])[4] == 0
    assert runner._graph_key([StepEntry("a", list(range(40)), [3])]) is None and runner._graph_key([StepEntry("a", list(range(40)), [3])]) is None   # a place inside the portion
    many = [StepEntry(f"r{i}", [1, 2], [1]) for i in range(PORTION_ROWS + 1)]
    for entry in many:
        runner.cache.open(entry.request_id)
    assert runner._graph_key(many) is None and runner._graph_key(many) is None
    assert runner._graph_key([StepEntry("a", list(range(513)), [512])]) is None and runner._graph_key([StepEntry("a", list(range(513)), [512])]) is None
    runner.capture_portions = False
    assert runner._graph_key(step) is None
    # the GPU's time against the host's: a tiny model is always the host's; at Qwen3-8B sizes a step of 128 tokens is the GPU's
    import llmserver_amd.models  # noqa: F401
    from llmserver_amd.config import named_config
    from llmserver_amd.weights.random_init import build_model
    assert runner._host_bounds_a_step(512, 1024)
    runner.model, runner._host_bound = build_model(named_config("qwen3-8b")), {}
    runner.dtype = torch.bfloat16
    assert runner._host_bounds_a_step(16, 1024) and not runner._host_bounds_a_step(128, 1024) and not runner._host_bounds_a_step(32, 16384)
    runner.model, runner._host_bound = build_model(named_config("qwen3-1.7b")), {}
    assert runner._host_bounds_a_step(512, 1024)
