"""Captured steps (single tokens; small steps with portions of prompts) against the same steps run eagerly: every
replay is checked, with eager work (portions of other prompts) and synchronisations between the replays."""
import random

import pytest
import torch

from helpers import model_folder, random_tokens
from tiny_configs import CASES

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("case, n_live", [("A", 3), ("B", 3), ("B", 5), ("B", 12), ("B", 21), ("B", 24)])
def test_replayed_steps_equal_eager_steps(case, n_live, dtype):
    """Three and twelve rows keep the products in the hand-written few-row kernels (one and two rows per
    wavefront in their fused epilogues); twenty-four rows put the library's products inside the captured graph; five
    and twenty-one rows are filled up to six and twenty-four with rows of nobody's (and, every ninth turn, three and
    eleven to three and twelve)."""
    from llmserver_amd.cache import CacheManager
    from llmserver_amd.engine import ModelRunner, StepEntry, load_model
    print(f"graph replay {case} {n_live} rows {dtype}", flush=True)
    raw, _, page = CASES[case]
    model = load_model(model_folder(case), "cuda", dtype)
    runners = []
    for use_graphs in (True, False):
        cache = CacheManager(model.cache_specs(), page, 500, device="cuda", dtype=model.dtype)
        runners.append(ModelRunner(model, cache, use_graphs=use_graphs))
        runners[-1].capture_portions = False       # (the portions between the replays are meant to be eager work here)
    lengths = [37, 5, 64, 1, 90, 16, 17, 33, 2, 70, 48, 9, 3, 81, 40, 7, 66, 21, 12, 55, 30, 8, 19, 44][:n_live]
    prompts = {f"r{i}": random_tokens(raw["vocab_size"], n, 1 + i) for i, n in enumerate(lengths)}
    feed = {rid: random_tokens(raw["vocab_size"], 80, 10 + i) for i, rid in enumerate(prompts)}
    for runner in runners:
        for rid, tokens in prompts.items():
            runner.cache.open(rid)
            runner.step([StepEntry(rid, tokens, [])])
    worst = 0.0
    for turn in range(70):
        live = list(prompts) if turn % 9 else list(prompts)[::2]        # another number of rows now and then: another graph
        entries = [StepEntry(rid, [feed[rid][turn]], [0]) for rid in live]
        outs = [runner.step(entries).clone() for runner in runners]
        torch.cuda.synchronize()
        worst = max(worst, float((outs[0] - outs[1]).abs().max()))
        if turn % 7 == 3:                                              # eager work between the replays
            for runner in runners:
                runner.cache.open("tmp")
                runner.step([StepEntry("tmp", random_tokens(raw["vocab_size"], 23, turn), [22])])
                runner.cache.close("tmp")
    assert runners[0].graph_replays >= 60 and runners[1].graph_replays == 0
    assert runners[0].graph_count() <= 3, list(runners[0]._graphs)     # both numbers of rows, and the prompt of one token
    assert worst <= (1e-5 if dtype == "float32" else 2e-2), worst
    for runner in runners:
        runner.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_prepared_ahead_equal_steps_prepared_in_time(dtype):
    """A decoding step whose host work was done before its tokens were known gives what the same step gives when
    it is prepared the usual way; a step that turns out to be another one than the one prepared (other requests,
    another order, a portion of a prompt between) drops what was prepared and is right all the same."""
    from llmserver_amd.cache import CacheManager
    from llmserver_amd.engine import ModelRunner, StepEntry, load_model
    case = "B"
    raw, _, page = CASES[case]
    model = load_model(model_folder(case), "cuda", dtype)
    runners = []
    for _ in range(2):
        cache = CacheManager(model.cache_specs(), page, 400, device="cuda", dtype=model.dtype)
        runners.append(ModelRunner(model, cache, use_graphs=True))
    ahead, plain = runners
    lengths = [37, 5, 64, 1, 90, 16, 17]
    prompts = {f"r{i}": random_tokens(raw["vocab_size"], n, 1 + i) for i, n in enumerate(lengths)}
    feed = {rid: random_tokens(raw["vocab_size"], 60, 10 + i) for i, rid in enumerate(prompts)}
    for runner in runners:
        for rid, tokens in prompts.items():
            runner.cache.open(rid)
            runner.step([StepEntry(rid, tokens, [])])
    worst, prepared = 0.0, 0
    for turn in range(60):
        live = list(prompts)
        if turn % 10 == 4:
            live = live[::2]                    # fewer requests than were prepared for
        if turn % 10 == 7:
            live = live[::-1]                   # the same requests in another order
        entries = [StepEntry(rid, [feed[rid][turn]], [0]) for rid in live]
        outs = [runner.step(entries).clone() for runner in runners]
        torch.cuda.synchronize()
        worst = max(worst, float((outs[0] - outs[1]).abs().max()))
        if turn % 10 == 8:                      # a portion of another prompt between the preparation and the step
            prepared += ahead.prepare_ahead(list(prompts))
            for runner in runners:
                runner.cache.open("tmp")
                runner.step([StepEntry("tmp", random_tokens(raw["vocab_size"], 23, turn), [22])])
                runner.cache.close("tmp")
        prepared += ahead.prepare_ahead(list(prompts))
    assert prepared >= 55                       # all but the first steps of a shape, which are captured the usual way
    assert 35 <= ahead.steps_prepared_ahead < prepared and plain.steps_prepared_ahead == 0
    assert worst <= (1e-5 if dtype == "float32" else 2e-2), worst
    assert not ahead.prepare_ahead(["nobody"]) and not ahead.prepare_ahead([]) and not ahead.prepare_ahead(["r0", "r0"])
    for runner in runners:
        runner.cache.check_invariants()
        for rid in prompts:
            runner.cache.close(rid)
        runner.cache.check_invariants()
        assert all(group.pool.num_available == group.pool.num_pages for group in runner.cache.groups)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_started_ahead_of_their_tokens_equal_steps_started_in_time(dtype):
    """Greedy decoding in which every step is started with the tokens of the step before still on the device, against
    the same decoding step by step; now and then the step that follows is another one than the one started (a request
    leaves, a portion of another prompt comes between), which must drop it and change nothing."""
    from llmserver_amd.cache import CacheManager
    from llmserver_amd.engine import ModelRunner, StepEntry, load_model
    case = "B"
    raw, _, page = CASES[case]
    model = load_model(model_folder(case), "cuda", dtype)
    runners = []
    for _ in range(2):
        cache = CacheManager(model.cache_specs(), page, 400, device="cuda", dtype=model.dtype)
        runners.append(ModelRunner(model, cache, use_graphs=True))
    ahead, plain = runners
    lengths = [37, 5, 64, 1, 90, 16]
    prompts = {f"r{i}": random_tokens(raw["vocab_size"], n, 1 + i) for i, n in enumerate(lengths)}
    last = {}
    for runner in runners:
        for rid, tokens in prompts.items():
            runner.cache.open(rid)
            logits = runner.step([StepEntry(rid, tokens, [len(tokens) - 1])])
            last[rid] = int(logits[0].argmax())
    live = list(prompts)
    worst = 0.0
    for turn in range(50):
        if turn == 20:
            live = live[:-1]                    # a request leaves after a step was started with it
        entries = [StepEntry(rid, [last[rid]], [0]) for rid in live]
        got, want = ahead.step(entries), plain.step(entries)
        worst = max(worst, float((got - want).abs().max()))
        sampled = want.argmax(dim=-1).to(torch.int32)       # both runners go on with the same tokens
        if turn % 10 == 6:                      # a portion of another prompt between the start and the step
            assert ahead.prepare_ahead(live) and ahead.launch_ahead(sampled)
            for runner in runners:
                runner.cache.open("tmp")
                runner.step([StepEntry("tmp", random_tokens(raw["vocab_size"], 23, turn), [22])])
                runner.cache.close("tmp")
        elif turn >= 2:
            assert ahead.prepare_ahead(live) and ahead.launch_ahead(sampled)
            assert not ahead.launch_ahead(sampled)          # nothing is prepared any more
        for rid, token in zip(live, sampled.tolist()):
            last[rid] = token
    assert ahead.steps_launched_ahead >= 45 and plain.steps_launched_ahead == 0
    assert worst <= (1e-5 if dtype == "float32" else 2e-2), worst
    for runner in runners:
        runner.cache.check_invariants()
        for rid in prompts:
            runner.cache.close(rid)
        assert all(group.pool.num_available == group.pool.num_pages for group in runner.cache.groups)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", ["B", "D"])
def test_replayed_steps_with_portions_equal_eager_steps(case, dtype):
    """Small steps that bring portions of prompts (alone, several, beside decoded tokens) are captured when their shape
    has been met twice and replayed afterwards, filled up with rows and tokens of nobody's; whatever the portions'
    lengths inside a shape, every step gives what the same step gives eagerly (where long rows go through other
    kernels and key ranges are cut otherwise), also after pages were given back and used again, with the library's
    products inside the graphs and eager steps between the replays."""
    from llmserver_amd.cache import CacheManager
    from llmserver_amd.engine import ModelRunner, StepEntry, load_model
    print(f"graph replay of steps with portions {case} {dtype}", flush=True)
    raw, _, page = CASES[case]
    vocab = raw["vocab_size"]
    model = load_model(model_folder(case), "cuda", dtype)
    runners = []
    for use_graphs in (True, False):
        cache = CacheManager(model.cache_specs(), page, 300, device="cuda", dtype=model.dtype)
        runners.append(ModelRunner(model, cache, use_graphs=use_graphs))
    captured, eager = runners
    rng = random.Random(11)
    decoders = {f"d{i}": random_tokens(vocab, n, 1 + i) for i, n in enumerate((37, 5, 64, 1))}
    feed = {rid: random_tokens(vocab, 200, 10 + i) for i, rid in enumerate(decoders)}
    for runner in runners:
        for rid, tokens in decoders.items():
            runner.cache.open(rid)
            runner.step([StepEntry(rid, tokens, [])])
    prompts, fed, opened, worst, scale, compared = {}, {}, 0, 0.0, 0.0, 0
    for turn in range(150):
        while len(prompts) < 2:                                        # two prompts under way at any time
            rid = f"p{opened}"
            prompts[rid], fed[rid] = random_tokens(vocab, rng.choice((9, 30, 64, 100, 150)), 100 + opened), 0
            opened += 1
            for runner in runners:
                runner.cache.open(rid)
        entries = [StepEntry(rid, [feed[rid][turn]], [0]) for rid in rng.sample(sorted(decoders), rng.choice((0, 0, 1, 2, 4)))]
        ended = []
        for rid in sorted(prompts)[:rng.choice((1, 1, 2))]:
            size = min(len(prompts[rid]) - fed[rid], rng.choice((2, 3, 7, 16, 31, 40)))
            reaches_end = fed[rid] + size == len(prompts[rid])
            entries.append(StepEntry(rid, prompts[rid][fed[rid]:fed[rid] + size], [size - 1] if reaches_end else []))
            fed[rid] += size
            if reaches_end:
                ended.append(rid)
        outs = [runner.step(entries).clone() for runner in runners]
        torch.cuda.synchronize()
        assert outs[0].shape == outs[1].shape == (sum(len(entry.want) for entry in entries), vocab)
        if outs[1].numel():
            worst, scale, compared = max(worst, float((outs[0] - outs[1]).abs().max())), max(scale, float(outs[1].abs().max())), compared + 1
        for rid in ended:                                               # its pages go back and are used again by the next prompts
            del prompts[rid]
            for runner in runners:
                runner.cache.close(rid)
        if turn % 11 == 5:                                             # an eager step between the replays: too many tokens to be captured
            for runner in runners:
                runner.cache.open("long")
                runner.step([StepEntry("long", random_tokens(vocab, 600, turn), [599])])
                runner.cache.close("long")
    kinds = [key[0] for key in captured._graphs]
    print(f"  {captured.graph_replays} replays of {len(kinds)} graphs ({kinds.count('portions')} with portions); worst difference {worst:.2e} "
          f"of logits up to {scale:.2e} in {compared} steps", flush=True)
    assert kinds.count("portions") >= 4 and captured.graph_replays >= 60 and eager.graph_replays == 0
    assert worst <= (2e-5 if dtype == "float32" else 1.5e-2) * scale, (worst, scale)
    for runner in runners:
        runner.cache.check_invariants()
