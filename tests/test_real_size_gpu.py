"""Two decoder layers at the real sizes of Qwen3-8B (width 4096, 32/8 heads of 128, intermediate
12288, vocabulary 151936, tied head to keep the folder small) against the plain implementation:
whole, in portions and token by token, in float32 and in bfloat16.  At these sizes a
reduced-precision matrix mode on the 32-bit path would show at once, and the products that depend
on the size run as in serving: the portion of 40 tokens leaves the results of both projections
into the residual stream as partial sums (two layers, so that the feed-forward's has a norm after it)."""
import numpy as np
import pytest
import torch

import plain_qwen3 as plain
from helpers import random_tokens
from llmserver_amd.config import config_from_dict
from llmserver_amd.weights import RandomInit, write_random_model

pytestmark = pytest.mark.gpu

REAL = dict(model_type="qwen3", num_hidden_layers=2, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8,
            head_dim=128, intermediate_size=12288, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
            attention_bias=False, tie_word_embeddings=True)


@pytest.fixture(scope="module")
def real_model(tmp_path_factory):
    folder = str(tmp_path_factory.mktemp("real_size"))
    write_random_model(config_from_dict(dict(REAL)), folder, RandomInit(seed=2, std=0.02, norm_noise=0.1))
    config, tensors = plain.read_folder(folder, dtype=torch.float32)
    tokens = random_tokens(REAL["vocab_size"], 83, 77)
    with torch.no_grad():
        expected = plain.forward(config, tensors, tokens).numpy()
    del tensors
    return folder, tokens, expected


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_real_size_layer_matches_the_plain_implementation(real_model, dtype):
    from llmserver_amd.cache import CacheManager
    from llmserver_amd.engine import ModelRunner, StepEntry, load_model
    print(f"real size layer {dtype}", flush=True)
    folder, tokens, expected = real_model
    model = load_model(folder, "cuda", dtype)
    cache = CacheManager(model.cache_specs(), 16, 24, device="cuda", dtype=model.dtype)
    runner = ModelRunner(model, cache)
    scale = float(np.abs(expected).max())
    limit = 2e-4 * scale if dtype == "float32" else 0.03 * scale
    schedules = {"whole": [(0, 83)], "portions": [(0, 40), (40, 42), (42, 75), (75, 83)],
                 "tail": [(0, 70)] + [(p, p + 1) for p in range(70, 83)]}
    for name, cuts in schedules.items():
        cache.open(name)
        rows = []
        for start, end in cuts:
            rows.append(runner.step([StepEntry(name, tokens[start:end], list(range(end - start)))]).float().cpu().numpy())
        cache.close(name)
        got = np.concatenate(rows)
        error = float(np.abs(got - expected).max())
        assert error <= limit, f"{name}: {error} > {limit} (logit scale {scale})"
    cache.check_invariants()
