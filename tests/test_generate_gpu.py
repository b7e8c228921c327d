"""Generation through the Python entry point and the engine on the GPU."""
import pytest
import torch

import plain_qwen3 as plain
from helpers import model_folder, plain_model, random_tokens
from tiny_configs import CASES

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("case", ["A", "C"])
def test_greedy_generation_matches_the_plain_implementation(case):
    """Workload of tiny configuration A: prompts of 5, 17 and 33 tokens, 8 greedy tokens each."""
    from llmserver_amd import generate
    print(f"greedy generation case {case}", flush=True)
    config, tensors = plain_model(case)
    prompts = [random_tokens(config["vocab_size"], n, 40 + i) for i, n in enumerate((5, 17, 33))]
    expected = [plain.greedy_generate(config, tensors, prompt, 8) for prompt in prompts]
    got = generate(model_folder(case), prompts, max_new_tokens=8, dtype="float32", block_size=CASES[case][2])
    assert got == expected
    got_bf16 = generate(model_folder(case), prompts, max_new_tokens=8, dtype="bfloat16", block_size=CASES[case][2])
    agree = sum(a == b for g, e in zip(got_bf16, expected) for a, b in zip(g, e))
    assert agree >= 20, (got_bf16, expected)             # bfloat16 may leave the greedy path where two logits nearly tie


@pytest.mark.parametrize("case", ["A", "B"])
def test_engine_with_its_default_pages_of_500_tokens(case):
    """The engine's own defaults (500 pages of 500 tokens, as the reference's engine has them): prompts that end
    inside the first page and one that crosses into a second, decoded past the page's edge."""
    from llmserver_amd import Engine, load_model
    print(f"engine with default pages, case {case}", flush=True)
    config, tensors = plain_model(case)
    prompts = [random_tokens(config["vocab_size"], n, 70 + i) for i, n in enumerate((3, 40, 493, 620))]
    expected = [plain.greedy_generate(config, tensors, prompt, 12) for prompt in prompts]
    engine = Engine(load_model(model_folder(case), "cuda", "float32"), None, max_new_tokens=12, max_batch_size=4, ignore_eos=True)
    assert engine.block_size == 500
    assert engine.generate(prompts) == expected
    engine.kv_cache.check_invariants()
    # In bfloat16 the kernel that shares a workgroup's keys between its tiles takes pages of a multiple of 8 keys: with
    # the default of 500 prompts go through the per-tile kernel instead, and the engine says so when it is made.
    import warnings
    model = load_model(model_folder(case), "cuda", "bfloat16")
    with pytest.warns(UserWarning, match="multiple of 8 keys"):
        slow = Engine(model, None, max_new_tokens=12, max_batch_size=4, ignore_eos=True)
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        fast = Engine(model, None, max_new_tokens=12, max_batch_size=4, ignore_eos=True, kv_cache_block_size=496)
    agree = sum(a == b for got, other in zip(slow.generate(prompts), fast.generate(prompts)) for a, b in zip(got, other))
    assert agree >= 40, agree            # (two roundings of the same model: greedy paths part only where two logits nearly tie)


@pytest.mark.parametrize("case", ["A", "B", "C"])
@pytest.mark.parametrize("rows", [5, 12, 16, 24])
def test_wide_decode_steps_match_the_plain_implementation(case, rows):
    """One step that decodes a token for each of 5, 12, 16 or 24 requests at once (bfloat16): up to 16 rows the
    few-row products carry the sums and norms between them in their epilogues (one row per wavefront up to 8, two
    beyond), 24 rows go through the library's products and the separate kernels; every row must give the plain
    implementation's logits for its own sequence."""
    from helpers import check_against_rounded_oracle, plain_logits, relative_error, rounded_logits
    from llmserver_amd.cache import CacheManager
    from llmserver_amd.engine import ModelRunner, StepEntry, load_model
    print(f"wide decode step {case} {rows} rows", flush=True)
    raw, _, page = CASES[case]
    model = load_model(model_folder(case), "cuda", "bfloat16")
    cache = CacheManager(model.cache_specs(), page, 400, device="cuda", dtype=model.dtype)
    runner = ModelRunner(model, cache, use_graphs=False)
    lengths = [37, 5, 64, 2, 90, 16, 17, 33, 3, 70, 48, 9, 4, 81, 40, 7, 66, 21, 12, 55, 30, 8, 19, 44][:rows]
    tokens = {f"r{i}": random_tokens(raw["vocab_size"], n, 300 + i) for i, n in enumerate(lengths)}
    for rid, sequence in tokens.items():
        cache.open(rid)
        runner.step([StepEntry(rid, sequence[:-1], [])])
    logits = runner.step([StepEntry(rid, sequence[-1:], [0]) for rid, sequence in tokens.items()]).float().cpu().numpy()
    # the rows' errors against what the rounded oracle loses anywhere in these sequences (a row is one place of its sequence)
    errors = [relative_error(logits[i], plain_logits(case, n, 300 + i)[n - 1].numpy()) for i, n in enumerate(lengths)]
    lost = [relative_error(row, exact) for i, n in enumerate(lengths)
            for row, exact in zip(rounded_logits(case, n, 300 + i).numpy(), plain_logits(case, n, 300 + i).numpy())]
    check_against_rounded_oracle(errors, lost, f"{rows} decoded rows in one step")
    cache.check_invariants()


def test_small_budget_and_few_pages_give_the_same_tokens():
    """Chunked prefill beside decodes under a token budget of 32, and a pool so small that requests
    are preempted and recomputed, must not change greedy output (float32)."""
    from llmserver_amd import Engine, load_model
    print("generation under a small budget", flush=True)
    case = "B"
    config, tensors = plain_model(case)
    prompts = [random_tokens(config["vocab_size"], n, 60 + i) for i, n in enumerate((1, 40, 64, 100))]
    expected = [plain.greedy_generate(config, tensors, prompt, 12) for prompt in prompts]
    model = load_model(model_folder(case), "cuda", "float32")
    roomy = Engine(model, None, max_new_tokens=12, max_batch_size=4, max_num_batched_tokens=32, kv_cache_num_blocks=64,
                   kv_cache_block_size=8, ignore_eos=True)
    assert roomy.generate(prompts) == expected
    tight = Engine(model, None, max_new_tokens=12, max_batch_size=4, max_num_batched_tokens=32, kv_cache_num_blocks=27,
                   kv_cache_block_size=8, ignore_eos=True)
    assert tight.generate(prompts) == expected
    assert tight.step_profile["preemptions"] > 0
    tight.kv_cache.check_invariants()
    assert min(tight.kv_cache.available_pages()) == 27


def test_graphs_captured_ahead_change_nothing():
    """Decode graphs captured before serving: all pages come back, and generation gives the tokens it gives without
    (greedy, bfloat16, several requests at once so that the captured sizes are met)."""
    from llmserver_amd import Engine, load_model
    print("graphs captured ahead", flush=True)
    case = "A"
    raw, _, page = CASES[case]
    prompts = [random_tokens(raw["vocab_size"], n, 80 + i) for i, n in enumerate((5, 17, 33, 9))]
    model = load_model(model_folder(case), "cuda", "bfloat16")
    def engine():
        return Engine(model, None, max_new_tokens=10, max_batch_size=4, max_num_batched_tokens=64, kv_cache_num_blocks=40,
                      kv_cache_block_size=page, ignore_eos=True)
    plain_run = engine().generate(prompts)
    warmed = engine()
    assert warmed.warmup_graphs() == 5                                   # 1, 2, 3 and 4 rows of short contexts; 1 row beyond them
    assert min(warmed.kv_cache.available_pages()) == 40 and not warmed.kv_cache.requests
    replays = warmed.runner.graph_replays
    assert warmed.generate(prompts) == plain_run
    assert warmed.runner.graph_replays > replays and warmed.runner.graph_count() == 5     # no further capture was needed
    # decoding steps were laid out, most of them also started, while the step before them ran
    assert warmed.runner.steps_prepared_ahead + warmed.runner.steps_launched_ahead >= 6 and warmed.runner.steps_launched_ahead >= 3
    assert min(warmed.kv_cache.available_pages()) == 40 and not warmed.kv_cache.requests
    warmed.add_request(None, prompt_token_ids=[1, 2, 3])
    assert warmed.warmup_graphs() == 0                                   # not while requests are live
    warmed.kv_cache.check_invariants()
    # longer contexts: a graph for every width of the block table up to the context, where the pool can hold the rows
    roomy = Engine(model, None, max_new_tokens=10, max_batch_size=4, max_num_batched_tokens=64, kv_cache_num_blocks=200,
                   kv_cache_block_size=page, ignore_eos=True)
    # 1, 2, 4 rows of short contexts, the same beyond them, 1 and 2 rows behind 64 pages
    assert roomy.warmup_graphs(batch_sizes=(1, 2, 4), max_context=64 * page + 70) == 8
    assert sorted((key[0], key[1], key[3] == ("short contexts",)) for key in roomy.runner._graphs) == [
        (1, 64, False), (1, 64, True), (1, 128, False), (2, 64, False), (2, 64, True), (2, 128, False), (4, 64, False), (4, 64, True)]
    assert min(roomy.kv_cache.available_pages()) == 200 and not roomy.kv_cache.requests
    assert roomy.generate(prompts) == plain_run
    roomy.kv_cache.check_invariants()


def test_temperature_sampling_is_seeded_per_request():
    """Workload of tiny configuration B: temperature 0.8 with a fixed seed; a request's tokens do not
    depend on what shares its batch or on the token budget."""
    from llmserver_amd import Engine, load_model
    print("temperature sampling", flush=True)
    case = "B"
    vocab = CASES[case][0]["vocab_size"]
    prompts = [random_tokens(vocab, n, 80 + i) for i, n in enumerate((1, 40, 64, 100))]
    model = load_model(model_folder(case), "cuda", "float32")

    def run(budget, batch, which):
        engine = Engine(model, None, max_new_tokens=12, max_batch_size=batch, max_num_batched_tokens=budget,
                        kv_cache_num_blocks=64, kv_cache_block_size=8, ignore_eos=True, temperature=0.8)
        requests = [engine.add_request(None, prompts[i], seed=1000 + i) for i in which]
        while engine.step():
            pass
        return {i: r.generated_token_ids for i, r in zip(which, requests)}

    together = run(32, 4, [0, 1, 2, 3])
    alone = {}
    for i in range(4):
        alone.update(run(256, 1, [i]))
    assert together == alone
    assert len({tuple(v) for v in together.values()}) == 4
    other_seed = Engine(model, None, max_new_tokens=12, max_batch_size=1, max_num_batched_tokens=256, kv_cache_num_blocks=64,
                        kv_cache_block_size=8, ignore_eos=True, temperature=0.8)
    r = other_seed.add_request(None, prompts[3], seed=5)
    while other_seed.step():
        pass
    assert r.generated_token_ids != together[3]


def test_temperature_sampling_matches_the_plain_inverse_cdf():
    """Workload of tiny configuration B (prompts of 1, 40, 64 and 100 tokens under a budget of 32, 12 tokens each at
    temperature 0.8, a seed per request) in float32 against the plain implementation: every sampled token is the one
    that the request's own uniform number picks from softmax(logits / 0.8) of the plain logits over the request's
    sequence so far.  (The reference samples greedily only, utils/engine.py:295-297; stops and streaming as
    utils/engine.py:299-314.)  A wrong scale of the softmax, an edge off by one token or a number drawn for the wrong
    request or step moves most tokens.  The one exception has a name: a number within NEAR_AN_EDGE of the edge between
    two tokens may fall to either side (32-bit logits and running sums differ from the 64-bit ones in the sixth
    digit), and then the neighbouring token is demanded."""
    from llmserver_amd import Engine, load_model
    from llmserver_amd.sampling import request_uniform
    print("temperature sampling against the plain inverse CDF", flush=True)
    NEAR_AN_EDGE = 2e-5
    case, temperature, new_tokens = "B", 0.8, 12
    vocab = CASES[case][0]["vocab_size"]
    config, tensors = plain_model(case)
    prompts = [random_tokens(vocab, n, 80 + i) for i, n in enumerate((1, 40, 64, 100))]
    model = load_model(model_folder(case), "cuda", "float32")
    engine = Engine(model, None, max_new_tokens=new_tokens, max_batch_size=4, max_num_batched_tokens=32,
                    kv_cache_num_blocks=64, kv_cache_block_size=8, ignore_eos=True, temperature=temperature)
    requests = [engine.add_request(None, prompt, seed=1000 + i) for i, prompt in enumerate(prompts)]
    while engine.step():
        pass
    assert engine.step_profile["prefill_steps"] >= 7          # the budget cut the prompts into portions beside decodes
    near, greedy_agrees = 0, 0
    for i, (prompt, request) in enumerate(zip(prompts, requests)):
        generated = list(request.generated_token_ids)
        assert len(generated) == new_tokens
        for draw, token in enumerate(generated):
            logits = plain.forward(config, tensors, prompt + generated[:draw])[-1]
            uniform = request_uniform(1000 + i, draw)
            expected, margin = plain.inverse_cdf_sample(logits, temperature, uniform)
            greedy_agrees += token == int(torch.argmax(logits))
            if margin < NEAR_AN_EDGE:
                near += 1
                assert abs(token - expected) <= 1, (i, draw, token, expected, margin)
            else:
                assert token == expected, (i, draw, token, expected, margin)
    assert near <= 1, f"{near} of {4 * new_tokens} numbers fell next to an edge between two tokens"
    assert greedy_agrees < 2 * new_tokens                     # (the temperature did something: these are not the greedy tokens)


def test_engine_refuses_to_run_without_its_kernels(monkeypatch):
    """No CPU path: asking for the kernels where no GPU is visible raises instead of falling back."""
    from llmserver_amd.kernels import KernelLibraryMissing, ops
    monkeypatch.setattr(torch.cuda, "is_available", lambda: False)
    with pytest.raises(KernelLibraryMissing):
        ops.HipOps()


@pytest.mark.parametrize("places", [6, 3])
@pytest.mark.parametrize("temperature", [0.0, 0.8])
def test_steps_started_ahead_give_the_same_tokens_also_when_requests_stop_unforeseen(temperature, places):
    """Decoding steps are started before the host has seen the tokens they bring; an end-of-sequence token makes the
    step that was started another one than the step that follows.  Same tokens, same reasons to stop and every page
    back, with and without starting ahead (bfloat16, requests of different lengths, stops by token and by length)."""
    from llmserver_amd import Engine, load_model
    print(f"steps started ahead, temperature {temperature}, {places} places", flush=True)
    case = "A"
    raw, _, page = CASES[case]
    prompts = [random_tokens(raw["vocab_size"], n, 500 + i) for i, n in enumerate((5, 17, 33, 9, 2, 21))]
    limits = [40, 12, 40, 25, 40, 7]
    model = load_model(model_folder(case), "cuda", "bfloat16")
    def make(launch_ahead):
        # with three places for six requests some wait while the others decode: steps are started ahead all the same
        return Engine(model, None, max_new_tokens=40, max_batch_size=places, max_num_batched_tokens=128, kv_cache_num_blocks=60,
                      kv_cache_block_size=page, ignore_eos=False, temperature=temperature, seed=3, launch_ahead=launch_ahead)
    free_run = make(False)
    free = [free_run.add_request(None, prompt_token_ids=prompt, max_new_tokens=limit) for prompt, limit in zip(prompts, limits)]
    while free_run.step():
        pass
    # tokens that some requests produce in the middle of their run end those requests (and whoever else produces them)
    stops = {free[0].generated_token_ids[6], free[2].generated_token_ids[10], free[4].generated_token_ids[3]}
    outcomes = []
    for launch_ahead in (False, True):
        engine = make(launch_ahead)
        engine.eos_token_ids = set(stops)
        requests = [engine.add_request(None, prompt_token_ids=prompt, max_new_tokens=limit) for prompt, limit in zip(prompts, limits)]
        while engine.step():
            pass
        outcomes.append([(list(r.generated_token_ids), r.finish_reason) for r in requests])
        assert min(engine.kv_cache.available_pages()) == 60 and not engine.kv_cache.requests
        engine.kv_cache.check_invariants()
        assert (engine.runner.steps_launched_ahead > 0) == launch_ahead
    assert outcomes[0] == outcomes[1]
    reasons = {reason.value for _, reason in outcomes[1]}
    assert len(reasons) == 2, reasons                                        # some stopped by a token, some by their length


@pytest.mark.parametrize("case, seed", [("A", 0), ("B", 1), ("C", 2), ("B", 4)])
def test_requests_arriving_over_time_with_shared_prefixes_and_few_pages(case, seed):
    """Fourteen requests, half of them behind a common prefix, arrive while others run; places, token budget and
    pages are few (requests wait, prompts are cut, pages of finished requests are cached and used again, requests
    are preempted); steps are started ahead or not.  Greedy float32 tokens of every request against the plain
    implementation."""
    import random
    from llmserver_amd import Engine, load_model
    print(f"arrivals over time {case} {seed}", flush=True)
    raw, _, page = CASES[case]
    config, tensors = plain_model(case)
    model = load_model(model_folder(case), "cuda", "float32")
    rng = random.Random(seed)
    prefix = random_tokens(raw["vocab_size"], rng.choice((2 * page, 3 * page + 1, 5 * page)), 900 + seed)
    prompts, limits = [], []
    for i in range(14):
        body = random_tokens(raw["vocab_size"], rng.randint(1, 60), 1000 + 50 * seed + i)
        prompts.append(prefix + body if rng.random() < 0.5 else body)
        limits.append(rng.randint(1, 40))           # (long enough that running requests outgrow their spare pages on the tight pool)
    expected = [plain.greedy_generate(config, tensors, p, n) for p, n in zip(prompts, limits)]
    longest = max(len(p) + n for p, n in zip(prompts, limits))
    preemptions_on_the_tight_pool = hits = 0
    for launch_ahead in (True, False):
        for pages in (400, -(-longest // page) + rng.choice((1, 3, 8))):
            engine = Engine(model, None, max_new_tokens=40, max_batch_size=rng.choice((2, 4, 6)), max_num_batched_tokens=rng.choice((16, 32, 128)),
                            kv_cache_num_blocks=pages, kv_cache_block_size=page, ignore_eos=True, launch_ahead=launch_ahead)
            order, requests, steps = list(range(len(prompts))), {}, 0
            while order or engine.scheduler.waiting or engine.scheduler.running:
                for _ in range(rng.choice((0, 1, 1, 3))):
                    if order:
                        i = order.pop(0)
                        requests[i] = engine.add_request(None, prompt_token_ids=prompts[i], max_new_tokens=limits[i])
                if engine.scheduler.waiting or engine.scheduler.running:
                    engine.step()
                    steps += 1
                assert steps < 2000
            engine.kv_cache.check_invariants()
            assert min(engine.kv_cache.available_pages()) == pages and not engine.kv_cache.requests
            for i in range(len(prompts)):
                assert list(requests[i].generated_token_ids) == expected[i], (launch_ahead, pages, i)
            assert pages < 400 or engine.step_profile["preemptions"] == 0
            preemptions_on_the_tight_pool += engine.step_profile["preemptions"] if pages < 400 else 0
            hits += engine.step_profile["prefix_hit_tokens"]
    assert hits > 0
    assert preemptions_on_the_tight_pool > 0, "the tight pool (the longest request and a few pages) preempted nobody"


def test_calibrate_measures_only_when_asked_and_writes_a_table(tmp_path):
    """Serving looks kernel choices up; ``Engine.calibrate`` is the one place that measures, and it leaves a file that a
    later process can be pointed at."""
    import json
    from llmserver_amd import Engine, load_model
    from llmserver_amd.kernels import default_ops
    from llmserver_amd.kernels.choices import ChoiceTable
    print("calibrate", flush=True)
    ops = default_ops()
    saved, ops.choices = ops.choices, ChoiceTable(ops.device_kind)
    try:
        model = load_model(model_folder("B"), "cuda", "bfloat16")
        engine = Engine(model, None, max_new_tokens=4, max_batch_size=3, max_num_batched_tokens=64, kv_cache_num_blocks=64, kv_cache_block_size=8)
        assert engine.generate([[1, 2, 3], [4, 5]]) and not ops.choices.entries       # generation measured nothing
        path = str(tmp_path / "choices.json")
        measured = engine.calibrate(save_to=path)
        assert measured > 0 and len(ops.choices.measured) == measured and ops._flush is None
        stored = json.load(open(path))
        assert list(stored) == [ops.device_kind] and len(stored[ops.device_kind]) == measured
        assert engine.generate([[1, 2, 3], [4, 5]])
        assert engine.calibrate() == 0                                                # everything is known now
    finally:
        ops.choices = saved
