"""A context of a few thousand tokens with attention made sharp, so that single far keys decide the result: the
per-head norm weights of q and k are scaled up, scores then spread over a dozen units and every query's softmax rests
on a handful of keys anywhere in its past.  A key lost, doubled or read from the wrong page (at a table chunk's edge,
in a key range's last step, in a page used again) moves the logits by far more than rounding does.  Through the
replay code: whole, in large portions (the workgroup-tile kernel, with and without keys before the portion), the tail
token by token (split key ranges and their merge), and beside other requests whose pages are used again."""
import io

import numpy as np
import pytest
import torch
from safetensors.torch import load_file, save_file

import plain_qwen3 as plain
import traces
from helpers import BF16, check_against_rounded_oracle, random_tokens, relative_error
from llmserver_amd.config import config_from_dict
from llmserver_amd.weights import RandomInit, write_random_model

pytestmark = pytest.mark.gpu

CONFIG = dict(model_type="qwen3", num_hidden_layers=2, hidden_size=256, num_attention_heads=10, num_key_value_heads=2, head_dim=64,
              intermediate_size=520, vocab_size=2003, rope_theta=1e6, rms_norm_eps=1e-6, attention_bias=False, tie_word_embeddings=True)
LENGTH = 2100
SHARPER = 2.0


@pytest.fixture(scope="module")
def sharp_model(tmp_path_factory):
    folder = str(tmp_path_factory.mktemp("sharp"))
    write_random_model(config_from_dict(dict(CONFIG)), folder, RandomInit(seed=17, std=0.02, norm_noise=0.1))
    path = f"{folder}/model.safetensors"
    tensors = load_file(path)
    for name in tensors:
        if name.endswith("q_norm.weight") or name.endswith("k_norm.weight"):
            tensors[name] = (tensors[name].float() * SHARPER).to(tensors[name].dtype)
    save_file(tensors, path)
    config, tensors = plain.read_folder(folder)
    main = random_tokens(CONFIG["vocab_size"], LENGTH, 41)
    others = {f"m{i}": random_tokens(CONFIG["vocab_size"], n, 50 + i) for i, n in enumerate((700, 64, 1300, 129, 300))}
    with torch.no_grad():
        expected = {"main": plain.forward(config, tensors, main).numpy()}
        expected.update({rid: plain.forward(config, tensors, tokens).numpy() for rid, tokens in others.items()})
        # what bfloat16 loses on these sequences (sharp scores make the rounding of q and k count): the rounded oracle
        lost = [relative_error(row, exact) for rid, tokens in dict(others, main=main).items()
                for row, exact in zip(plain.forward(config, tensors, tokens, r=BF16).numpy(), expected[rid])]
    return folder, main, others, expected, lost


def build_steps(main, others):
    steps, owner = [], {}

    def add(requests, maker, name_of):
        for step in maker(requests):
            step["step"] = len(steps)
            steps.append(step)
        owner.update(name_of)

    add({"w": main}, traces.whole, {"w": "main"})
    add({"t": main}, lambda r: traces.tail_decoded(r, 32), {"t": "main"})
    add({"p": main}, lambda r: traces.changing_portions(r, (700, 2, 130, 512, 17, 64, 33, 1000)), {"p": "main"})
    mixed = dict(others, q=main)
    add(mixed, lambda r: traces.mixed(r, seed=3, budget_tokens=traces.round64(LENGTH) + 1344 + 768), {**{k: k for k in others}, "q": "main"})
    return steps, owner


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sharp_attention_over_a_long_context(sharp_model, dtype, tmp_path, monkeypatch):
    from llmserver_amd.engine.replay import make_runner, replay
    print(f"sharp attention over {LENGTH} tokens, {dtype}", flush=True)
    folder, main, others, expected, lost = sharp_model
    steps, owner = build_steps(main, others)
    runner = make_runner(folder, dtype, traces.peak_tokens(steps), 16)
    out = str(tmp_path / "out")
    from llmserver_amd.parts import attention as attention_module
    plans, build = [], attention_module.build_attention_plan
    monkeypatch.setattr(attention_module, "build_attention_plan", lambda *args, **kwargs: plans.append(build(*args, **kwargs)) or plans[-1])
    assert replay(runner, traces.to_lines(steps).splitlines(), out, report=io.StringIO()) == len(steps)
    runner.cache.check_invariants()
    # what the steps went through: wavefronts with split key ranges, workgroups of tiles, and (bfloat16) workgroups
    # that share the keys of short portions behind the long context
    assert any(plan.n_slots and len(plan.items) for plan in plans) and any(len(plan.tiles) for plan in plans)
    assert (dtype == "bfloat16") == any(plan.tile_slots is not None for plan in plans)
    results = traces.collect(steps, out, CONFIG["vocab_size"])
    errors = {}
    for (rid, position), logits in results.items():
        want = expected[owner[rid]][position]
        errors.setdefault(rid, []).append(relative_error(logits, want))
    assert sum(len(v) for v in errors.values()) == 4 * LENGTH + sum(len(t) for t in others.values())
    worst = {rid: max(v) for rid, v in errors.items()}
    print("  worst by request:", {rid: f"{e:.2e}" for rid, e in worst.items()}, flush=True)
    if dtype == "float32":
        assert max(worst.values()) <= 3e-5, worst
    else:
        # rounding of q and k to 8 bits moves sharp scores by a tenth of a unit: several per cent of the largest logit
        # at the worst places, a per cent at the median, as the rounded oracle shows; a lost key moves them by tens of per cent
        check_against_rounded_oracle(np.concatenate([np.asarray(v) for v in errors.values()]), lost, "sharp attention")
        same_tokens = [relative_error(results[(other, p)], results[("w", p)]) for other in ("t", "p", "q") for p in range(LENGTH)]
        check_against_rounded_oracle(same_tokens, lost, "sharp attention, the same request cut in other ways", factor=2.0)
