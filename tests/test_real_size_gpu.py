"""Two decoder layers at the real sizes of Qwen3-8B (width 4096, 32/8 heads of 128, intermediate
12288, vocabulary 151936, tied head to keep the folder small) against the plain implementation:
whole, in portions and token by token, in float32 and in bfloat16.  At these sizes a
reduced-precision matrix mode on the 32-bit path would show at once, and the products that depend
on the size run as in serving: the portion of 40 tokens leaves the results of both projections
into the residual stream as partial sums (two layers, so that the feed-forward's has a norm after it).

A second test runs a mixed trace at these widths (a portion of 300 tokens and one of 40 beside 24 and 64 rows of one token
each, pages given back and used again), a third all 36 layers of Qwen3-8B once: what the depth does to bfloat16, and
to the 32-bit path, against the plain implementation run on the GPU.

The first two run at the widths of Qwen3-4B as well (2560, 32/8 heads, intermediate 9728: no powers of two, products
whose ranges of the inner dimension end in a shorter one, 20 tiles of weight rows where 8B has 32)."""
import random

import numpy as np
import pytest
import torch

import plain_qwen3 as plain
from helpers import BF16, check_against_rounded_oracle, random_tokens, relative_error
from llmserver_amd.config import config_from_dict
from llmserver_amd.weights import RandomInit, write_random_model

pytestmark = pytest.mark.gpu

REAL = dict(model_type="qwen3", num_hidden_layers=2, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8,
            head_dim=128, intermediate_size=12288, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
            attention_bias=False, tie_word_embeddings=True)


OTHER_WIDTHS = dict(REAL, hidden_size=2560, intermediate_size=9728)


@pytest.fixture(scope="module", params=[REAL, OTHER_WIDTHS], ids=["widths of 8B", "widths of 4B"])
def real_model(request, tmp_path_factory):
    folder = str(tmp_path_factory.mktemp("real_size"))
    write_random_model(config_from_dict(dict(request.param)), folder, RandomInit(seed=2, std=0.02, norm_noise=0.1))
    config, tensors = plain.read_folder(folder, dtype=torch.float32)
    tokens = random_tokens(REAL["vocab_size"], 83, 77)
    with torch.no_grad():
        expected = plain.forward(config, tensors, tokens).numpy()
        lost = [relative_error(row, exact) for row, exact in zip(plain.forward(config, tensors, tokens, r=BF16).numpy(), expected)]
    del tensors
    return folder, tokens, expected, lost


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_real_size_layer_matches_the_plain_implementation(real_model, dtype):
    from llmserver_amd.cache import CacheManager
    from llmserver_amd.engine import ModelRunner, StepEntry, load_model
    print(f"real size layer {dtype}", flush=True)
    folder, tokens, expected, lost = real_model
    model = load_model(folder, "cuda", dtype)
    cache = CacheManager(model.cache_specs(), 16, 24, device="cuda", dtype=model.dtype)
    runner = ModelRunner(model, cache)
    schedules = {"whole": [(0, 83)], "portions": [(0, 40), (40, 42), (42, 75), (75, 83)],
                 "tail": [(0, 70)] + [(p, p + 1) for p in range(70, 83)]}
    for name, cuts in schedules.items():
        cache.open(name)
        rows = []
        for start, end in cuts:
            rows.append(runner.step([StepEntry(name, tokens[start:end], list(range(end - start)))]).float().cpu().numpy())
        cache.close(name)
        errors = [relative_error(got, exact) for got, exact in zip(np.concatenate(rows), expected)]
        if dtype == "float32":
            assert max(errors) <= 2e-4, f"{name}: {max(errors)}"
        else:
            check_against_rounded_oracle(errors, lost, f"two layers at real size, {name}")
    cache.check_invariants()


def mixed_trace(vocab):
    """Steps (entries, ends) and every request's tokens: 72 short requests, a long one and a late one.

    0: 24 short prompts whole.  1: the first 300 tokens of the long request beside one token of each of the 24.
    2: eight of them have ended; 48 more short prompts and the long request's next 40 tokens.  3 to 5: 64 rows of one
    token each (a captured step, then replayed).  6: the long request's last token beside 16 rows.  7: everybody has
    ended; a late request of 140 tokens on their pages."""
    rng = random.Random(5)
    tokens = {f"d{i}": random_tokens(vocab, rng.choice((1, 2, 5, 9, 16, 17, 24)) + 5, 300 + i) for i in range(72)}
    tokens["long"] = random_tokens(vocab, 341, 401)
    tokens["late"] = random_tokens(vocab, 140, 402)
    fed = {rid: 0 for rid in tokens}

    def take(rid, count, want=None):
        start = fed[rid]
        fed[rid] = start + count
        return (rid, tokens[rid][start:start + count], [count - 1] if want is None else want)

    def prompt(rid):
        return take(rid, len(tokens[rid]) - 5)

    first, rest = [f"d{i}" for i in range(24)], [f"d{i}" for i in range(24, 72)]
    steps = [([prompt(rid) for rid in first], []),
             ([take("long", 300, [0, 137, 299])] + [take(rid, 1) for rid in first], first[:8]),
             ([prompt(rid) for rid in rest] + [take("long", 40, [0, 39])], [])]
    live = first[8:] + rest
    for _ in range(3):
        steps.append(([take(rid, 1) for rid in live], []))
    steps.append(([take("long", 1)] + [take(rid, 1) for rid in live[:16]], live + ["long"]))
    steps.append(([take("late", 140, [0, 70, 139])], ["late"]))
    return steps, tokens


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_steps_at_real_widths(real_model, dtype):
    """Products of 24, 40, 64, 140 and some 300 to 800 rows through the model at widths of 4,096 and 12,288 (the few-row
    kernels, the split products, the library whole and in ranges of the inner dimension), attention of prompt portions
    beside decoded tokens, and a pool that holds the peak and nothing more."""
    from llmserver_amd.cache import CacheManager
    from llmserver_amd.engine import ModelRunner, StepEntry, load_model
    print(f"real widths, mixed steps, {dtype}", flush=True)
    folder = real_model[0]
    steps, tokens = mixed_trace(REAL["vocab_size"])
    page = 16
    held, peak = {}, 0
    for entries, ends in steps:
        for rid, fed, _ in entries:
            held[rid] = held.get(rid, 0) + len(fed)
        peak = max(peak, sum(-(-n // page) for n in held.values()))
        for rid in ends:
            del held[rid]
    model = load_model(folder, "cuda", dtype)
    cache = CacheManager(model.cache_specs(), page, peak, device="cuda", dtype=model.dtype)
    runner = ModelRunner(model, cache)
    got, place = {}, {rid: 0 for rid in tokens}
    for entries, ends in steps:
        for rid, _, _ in entries:
            if not cache.has(rid):
                cache.open(rid)
        rows = runner.step([StepEntry(rid, fed, want) for rid, fed, want in entries]).float().cpu().numpy()
        row = 0
        for rid, fed, want in entries:
            for w in want:
                got[(rid, place[rid] + w)] = rows[row].copy()
                row += 1
            place[rid] += len(fed)
        for rid in ends:
            cache.close(rid)
    cache.check_invariants()
    assert min(cache.available_pages()) == peak and runner.graph_replays >= 2
    config, tensors = plain.read_folder(folder, dtype=torch.float32)
    errors, lost = [], []
    with torch.no_grad():
        for rid, sequence in tokens.items():
            places = sorted(p for r, p in got if r == rid)
            exact = plain.forward(config, tensors, sequence[:place[rid]], places=places).numpy()
            rounded = plain.forward(config, tensors, sequence[:place[rid]], places=places, r=BF16).numpy()
            for p, e, r in zip(places, exact, rounded):
                errors.append(relative_error(got[(rid, p)], e))
                lost.append(relative_error(r, e))
    assert len(errors) == 24 + 3 + 24 + 48 + 2 + 3 * 64 + 17 + 3
    print(f"  {dtype}: median {np.median(errors):.2e} worst {max(errors):.2e}", flush=True)
    if dtype == "float32":
        assert max(errors) <= 2e-4
    else:
        check_against_rounded_oracle(errors, lost, "mixed steps at real widths")


FULL_DEPTH = dict(REAL, num_hidden_layers=36, tie_word_embeddings=False)


def test_all_layers_at_real_size():
    """Qwen3-8B's 36 layers at their real sizes, random weights drawn on the GPU: a prompt of 512 tokens, then 16 tokens one
    by one, in bfloat16 and on the 32-bit path, against the plain implementation.  A 64-bit oracle of eight billion
    parameters on the CPU does not fit a test, so here the plain implementation runs on the GPU in float32 (the same
    functions, tensors on the device): that puts the oracle's own rounding near 1e-6, far below what bfloat16 loses, but
    it multiplies with the same library as the engine's 32-bit path, so a reduced-precision mode of that library would
    not show here (the two-layer tests above, whose oracle runs on the CPU, are where it shows).  Both runs have the
    same weights: values that bfloat16 holds."""
    from llmserver_amd.cache import CacheManager
    from llmserver_amd.engine import ModelRunner, StepEntry
    from llmserver_amd.weights.loader import stored_dtype
    from llmserver_amd.weights.random_init import build_model, random_tensor
    print("all 36 layers at real size", flush=True)
    config = config_from_dict(dict(FULL_DEPTH))
    init = RandomInit(seed=4, std=0.02, norm_noise=0.1)
    specs = build_model(config).param_specs()
    with torch.no_grad():
        oracle = {name: random_tensor(name, spec, init, device="cuda").to(stored_dtype(spec.role, torch.bfloat16)).float()
                  for name, spec in specs.items()}
    tokens = random_tokens(FULL_DEPTH["vocab_size"], 512 + 16, 91)
    places = [0, 1, 255, 256, 511] + list(range(512, 528))
    with torch.no_grad():
        exact = plain.forward(FULL_DEPTH, oracle, tokens, places=places).cpu().numpy()
        rounded = plain.forward(FULL_DEPTH, oracle, tokens, places=places, r=BF16).cpu().numpy()
    lost = [relative_error(r, e) for r, e in zip(rounded, exact)]
    for dtype in (torch.bfloat16, torch.float32):
        model = build_model(config)
        for name in specs:
            model.assign(name, oracle[name].to(stored_dtype(specs[name].role, dtype)))
        model.finalize(list(specs), "cuda", dtype)
        cache = CacheManager(model.cache_specs(), 16, 40, device="cuda", dtype=dtype)
        runner = ModelRunner(model, cache)
        cache.open("r")
        rows = [runner.step([StepEntry("r", tokens[:512], [0, 1, 255, 256, 511])]).float().cpu().numpy()]
        for position in range(512, 528):
            rows.append(runner.step([StepEntry("r", tokens[position:position + 1], [0])]).float().cpu().numpy())
        cache.close("r")
        cache.check_invariants()
        errors = [relative_error(g, e) for g, e in zip(np.concatenate(rows), exact)]
        print(f"  {dtype}: median {np.median(errors):.2e} worst {max(errors):.2e}; rounded oracle: median {np.median(lost):.2e} "
              f"worst {max(lost):.2e}", flush=True)
        if dtype == torch.float32:
            assert max(errors) <= 2e-4
        else:       # 21 places: the worst of them against the rounded oracle's worst
            check_against_rounded_oracle(errors, lost, "36 layers in bfloat16")
        del model, cache, runner
        torch.cuda.empty_cache()
