"""Seeded random configurations of the architecture (any number of heads and groups, head sizes in
steps of 16, widths, intermediate sizes and vocabularies that are no power of two and no multiple
of eight, every page size that divides 64) through the replay code against the plain
implementation: whole, last tokens one by one, changing portions and mixed with reused pages.
Each configuration runs in float32 and in bfloat16; the kernels have to take every one of them."""
import io
import os
import random

import numpy as np
import pytest
import torch

import plain_qwen3 as plain
import traces
from helpers import BF16, check_against_rounded_oracle, random_tokens, relative_error
from llmserver_amd.config import config_from_dict
from llmserver_amd.weights import RandomInit, write_random_model

pytestmark = pytest.mark.gpu

# The first nine are any seeds; the others are the ones at which wider runs of this same generator (some three hundred
# seeds) found the largest bfloat16 errors, 3 to 4.3 per cent of the logits, on narrow or deep configurations: one head of
# 160 over a width of 520 in four layers (7002), 35 heads of 16 over a width of 88 (0), a width of 12 (62), ...
SEEDS = (1, 2, 3, 5, 8, 13, 21, 34, 55, 0, 62, 71, 72, 158, 1001, 2013, 2032, 2036, 2049, 7002, 7003)


def random_config(rng):
    kv_heads = rng.choice((1, 1, 2, 2, 3, 4, 5, 8))
    group = rng.choice((1, 1, 2, 3, 4, 5, 7, 8))
    head_dim = 16 * rng.choice((1, 2, 3, 4, 4, 5, 6, 7, 8, 8, 10, 12, 16))
    hidden = rng.choice((24, 40, 56, 72, 88, 104, 136, 200, 264, 520, 100, 36, 1000, 20, 12))
    intermediate = rng.choice((24, 40, 100, 136, 200, 344, 520, 36, 1000, 44, 28))
    vocab = rng.choice((97, 256, 301, 1000, 1537, 5003, 33))
    return dict(model_type="qwen3", num_hidden_layers=rng.choice((1, 2, 3, 4)), hidden_size=hidden,
                num_attention_heads=kv_heads * group, num_key_value_heads=kv_heads, head_dim=head_dim,
                intermediate_size=intermediate, vocab_size=vocab,
                rope_theta=rng.choice((1e4, 5e4, 1e6, 123.0)), rms_norm_eps=rng.choice((1e-6, 1e-5, 1e-4)),
                attention_bias=rng.random() < 0.4, tie_word_embeddings=rng.random() < 0.5)


def random_trace(rng, vocab):
    steps, requests = [], {}

    def add(prefix, lengths, maker):
        made = {f"{prefix}{i}": random_tokens(vocab, n, rng.randrange(1 << 30)) for i, n in enumerate(lengths)}
        requests.update(made)
        for step in maker(made):
            step["step"] = len(steps)
            steps.append(step)

    long = rng.choice((257, 640, 900, 1300))
    add("w", [long, rng.randrange(1, 70)], traces.whole)
    add("t", [long], lambda r: traces.tail_decoded(r, 32))
    sizes = tuple(rng.choice((2, 3, 5, 7, 16, 17, 31, 33, 64, 100)) for _ in range(12))
    add("p", [long], lambda r: traces.changing_portions(r, sizes))
    lengths = [rng.choice((1, 2, 5, 17, 33, 64, 70, 100, 130, 200)) for _ in range(8)]
    add("m", lengths, lambda r: traces.mixed(r, seed=rng.randrange(1000), budget_tokens=rng.choice((256, 320, 512))))
    return steps, requests


ODD_WIDTHS = {"odd": dict(hidden_size=33, intermediate_size=25, vocab_size=101, head_dim=16, attention_bias=False),
              "few": dict(hidden_size=7, intermediate_size=5, vocab_size=3, head_dim=32, attention_bias=True),
              "one": dict(hidden_size=1, intermediate_size=1, vocab_size=2, head_dim=48, attention_bias=False),
              "wide": dict(hidden_size=129, intermediate_size=1027, vocab_size=7, head_dim=16, attention_bias=True)}


@pytest.mark.parametrize("name", sorted(ODD_WIDTHS))
def test_widths_that_no_vector_load_divides(name, tmp_path):
    """Widths, intermediate sizes and vocabularies that are odd or smaller than one vector load: rows then start at
    addresses that no wide load may assume, and the last partial vector must neither be dropped nor read past."""
    sizes = ODD_WIDTHS[name]
    raw = dict(model_type="qwen3", num_hidden_layers=2, num_attention_heads=3, num_key_value_heads=1, rope_theta=1e4,
               rms_norm_eps=1e-6, tie_word_embeddings=sizes["attention_bias"], **sizes)
    check_configuration(raw, 16, random.Random(len(name)), 7, tmp_path)


@pytest.mark.parametrize("seed", SEEDS)
def test_random_configuration_matches_the_plain_implementation(seed, tmp_path):
    rng = random.Random(seed)
    raw = random_config(rng)
    page_size = rng.choice((16, 16, 16, 4, 8, 32, 64))
    check_configuration(raw, page_size, rng, seed, tmp_path)


def check_configuration(raw, page_size, rng, seed, tmp_path):
    from llmserver_amd.engine.replay import make_runner, replay

    print(f"configuration {seed}: page {page_size} {raw}", flush=True)
    folder = str(tmp_path / "model")
    write_random_model(config_from_dict(dict(raw)), folder, RandomInit(seed=seed, std=rng.choice((0.02, 0.05, 0.1)), norm_noise=0.1))
    steps, requests = random_trace(rng, raw["vocab_size"])
    config, tensors = plain.read_folder(folder)
    expected = {rid: plain.forward(config, tensors, tokens).numpy() for rid, tokens in requests.items()}
    # what bfloat16 loses on this model and these tokens: the oracle that rounds where the reference's kernels round
    rounded = [relative_error(row, exact) for rid, tokens in requests.items()
               for row, exact in zip(plain.forward(config, tensors, tokens, r=BF16).numpy(), expected[rid])]
    for dtype in ("float32", "bfloat16"):
        runner = make_runner(folder, dtype, traces.peak_tokens(steps), page_size)
        out = str(tmp_path / dtype)
        assert replay(runner, traces.to_lines(steps).splitlines(), out, report=io.StringIO()) == len(steps)
        runner.cache.check_invariants()
        assert not runner.cache.requests, "every request of the trace was ended"
        results = traces.collect(steps, out, raw["vocab_size"])
        errors = np.asarray([relative_error(results[(rid, position)], expected[rid][position])
                             for rid, tokens in requests.items() for position in range(len(tokens))])
        assert np.isfinite(errors).all()
        print(f"  {dtype}: median {np.median(errors):.2e} worst {errors.max():.2e}", flush=True)
        if dtype == "float32":
            assert errors.max() <= 2e-5, f"{dtype}: {errors.max()} at {int(errors.argmax())}"
        else:
            check_against_rounded_oracle(errors, rounded, f"configuration {seed}")
        del runner
        torch.cuda.empty_cache()
