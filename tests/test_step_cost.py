"""What a step has to read and to multiply is summed over what the parts declare (``llmserver_amd.engine.cost``), not
written down per architecture: the sums equal the closed forms of the Qwen3 dense decoder, and the tests' toy
architectures (state of fixed size, windows, a block run twice, a cache read by a second call, experts of which a token
uses one) get theirs from the same functions."""
import dataclasses

import pytest
import torch

import test_toy_parts as toys
from llmserver_amd import models  # noqa: F401
from llmserver_amd.config import config_from_dict, named_config
from llmserver_amd.engine.cost import StepRow, cache_bytes, step_bytes, step_flops
from llmserver_amd.weights.random_init import build_model


def qwen3_closed_forms(c, elem):
    """Per layer: QKV, output, gate, up and down matrices; two norms of the width and two of the head size (float32)."""
    layer = c.hidden_size * (c.num_attention_heads + 2 * c.num_key_value_heads) * c.head_dim \
        + c.num_attention_heads * c.head_dim * c.hidden_size + 3 * c.hidden_size * c.intermediate_size
    vectors = 4 * (c.num_hidden_layers * (2 * c.hidden_size + 2 * c.head_dim) + c.hidden_size)
    kv_per_token = 2 * c.num_key_value_heads * c.head_dim * elem * c.num_hidden_layers
    return layer, vectors, kv_per_token


@pytest.mark.parametrize("name", ["qwen3-8b", "qwen3-1.7b", "tiny-b"])
def test_sums_over_the_parts_equal_the_closed_forms_of_the_dense_decoder(name):
    config = named_config(name)
    model = build_model(config)
    c = config
    for dtype, elem in ((torch.bfloat16, 2), (torch.float32, 4)):
        layer, vectors, kv_per_token = qwen3_closed_forms(c, elem)
        if name == "tiny-b":        # biases of q, k, v and the output projection (float32)
            vectors += 4 * c.num_hidden_layers * ((c.num_attention_heads + 2 * c.num_key_value_heads) * c.head_dim + c.hidden_size)
        # decoding: batch 8 at contexts 4,000 .. 4,007; every weight once, the head's too, an embedding row per token
        rows = [StepRow(1, 4000 + i) for i in range(8)]
        weights = elem * (c.num_hidden_layers * layer + c.vocab_size * c.hidden_size) + vectors + 8 * c.hidden_size * elem
        assert step_bytes(model, rows, dtype) == weights + kv_per_token * sum(4000 + i for i in range(8))
    # a prompt of 2,048 tokens: every matrix for every token, the head for one, causal attention
    tokens = 2048
    flops = 2.0 * tokens * layer * c.num_hidden_layers + 2.0 * c.vocab_size * c.hidden_size \
        + 2.0 * c.num_attention_heads * c.head_dim * tokens * (tokens + 1) * c.num_hidden_layers
    assert step_flops(model, [StepRow(tokens, tokens)]) == pytest.approx(flops, rel=1e-12)
    # a portion of 100 tokens behind 900: each of its tokens sees the 900 and its predecessors in the portion
    pairs = 100 * 900 + 100 * 101 // 2
    attention = 4.0 * c.num_attention_heads * c.head_dim * pairs * c.num_hidden_layers
    assert step_flops(model, [StepRow(100, 1000, wanted=0)]) == pytest.approx(2.0 * 100 * layer * c.num_hidden_layers + attention, rel=1e-12)


def toy_model(name):
    return build_model(config_from_dict(dict(toys.TOYS[name])))


def test_windows_state_and_the_order_of_calls_count_as_they_are_used():
    base = toys.BASE
    width, inter, d, heads, kv = base["hidden_size"], base["intermediate_size"], base["head_dim"], base["num_attention_heads"], base["num_key_value_heads"]
    kv_token = 2 * kv * d * 4
    rows = [StepRow(1, 100), StepRow(1, 5)]
    # windows of 9 and 20 beside layers that keep all keys: a context of 100 reads 100, 9, 20, 100, 9 keys
    assert cache_bytes(toy_model("windows"), rows, torch.float32) == kv_token * ((100 + 9 + 20 + 100 + 9) + (5 + 5 + 5 + 5 + 5))
    # a mixer with a state of `width` float32 numbers per request beside two attention layers
    assert cache_bytes(toy_model("state"), rows, torch.float32) == kv_token * 2 * 105 + 2 * width * 4
    # block 1 runs twice on caches of its own, and a fourth call reads the cache the first wrote: four reads of the keys,
    ordered = toy_model("order")
    assert cache_bytes(ordered, rows, torch.float32) == kv_token * 4 * 105
    # ... the weights of three blocks are read once each, and multiplied four times
    attention = width * (heads + 2 * kv) * d + heads * d * width
    block = attention + 3 * width * inter
    vectors = 4 * (3 * (2 * width + 2 * d) + width)
    embedding_rows, head = 2 * width * 4, base["vocab_size"] * width * 4
    assert step_bytes(ordered, rows, torch.float32) == 4 * 3 * block + vectors + embedding_rows + head + kv_token * 4 * 105
    mixing = 4.0 * heads * d * 105 * 4
    assert step_flops(ordered, rows) == pytest.approx(2.0 * 2 * 4 * block + 2.0 * 2 * base["vocab_size"] * width + mixing)
    # the running-mean mixer declares nothing between its projections
    assert toy_model("state").blocks[1].mixer.mixing_flops(7, 50) == 0.0
    # a window bounds the keys a token sees
    windowed = toy_model("windows").blocks[1].mixer
    assert windowed.mixing_flops(3, 30) == 4.0 * heads * d * 3 * 9 and windowed.mixing_flops(12, 12) == 4.0 * heads * d * (sum(range(1, 10)) + 3 * 9)


def test_a_tensor_of_which_a_token_uses_a_share_is_read_and_multiplied_by_that_share():
    """Experts of which every token uses one of four: a step of one token reads a quarter of their matrices, a step of
    many tokens nearly all of them (the expected share that some token uses), and every token multiplies a quarter."""
    model = toy_model("experts")
    dense = step_bytes(model, [StepRow(1, 10)], torch.float32), step_flops(model, [StepRow(1, 10)])
    block = model.blocks[1]
    specs = block.param_specs()
    expert_names = [name for name in specs if ".experts." in name]
    assert len(expert_names) == 9                       # three experts of three matrices each
    sizes = sum(torch.Size(specs[name].shape).numel() for name in expert_names)
    routed = {name: dataclasses.replace(spec, share_per_token=1 / 3 if name in expert_names else 1.0) for name, spec in specs.items()}
    block.param_specs = lambda: routed
    assert step_bytes(model, [StepRow(1, 10)], torch.float32) == pytest.approx(dense[0] - 4 * sizes * 2 / 3)
    assert step_flops(model, [StepRow(1, 10)]) == pytest.approx(dense[1] - 2.0 * sizes * 2 / 3)
    many = [StepRow(1, 10)] * 24
    assert step_bytes(model, many, torch.float32) == pytest.approx(step_bytes(toy_model("experts"), many, torch.float32) - 4 * sizes * (2 / 3) ** 24)
