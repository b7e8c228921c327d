"""Configuration, registry, weight loading errors and the random-weights mode (CPU)."""
import json
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

from llmserver_amd.config import (ConfigError, Qwen3Config, UnsupportedModelError, config_from_dict, load_config,
                                  registered_architectures)
from llmserver_amd.engine import load_model
from llmserver_amd.weights import RandomInit, WeightsError, build_model, write_random_model
from tiny_configs import CASES, TINY_A, TINY_B, make_config


def test_config_reads_its_own_keys_and_defaults():
    a, b = make_config(TINY_A), make_config(TINY_B)
    assert (a.num_hidden_layers, a.hidden_size, a.head_dim, a.group_size, a.tie_word_embeddings) == (2, 64, 16, 2, True)
    assert (b.num_attention_heads * b.head_dim, b.hidden_size, b.attention_bias, b.rms_norm_eps) == (256, 96, True, 1e-5)
    raw = {k: v for k, v in TINY_A.items() if k not in ("head_dim", "rope_theta")}
    c = config_from_dict(raw)
    assert c.head_dim == 64 // 4 and c.rope_theta == 10000.0            # reference defaults
    c = config_from_dict(dict(raw, rope_parameters={"rope_theta": 5e5}))
    assert c.rope_theta == 5e5
    c = config_from_dict({k: v for k, v in raw.items() if k != "num_key_value_heads"})
    assert c.num_key_value_heads == c.num_attention_heads == 4 and c.group_size == 1     # left out: multi-head attention
    # keys a published config.json of the architecture carries beside the ones that are read change nothing
    published = dict(TINY_A, architectures=["Qwen3ForCausalLM"], torch_dtype="bfloat16", sliding_window=None, use_sliding_window=False,
                     max_window_layers=2, rope_scaling=None, attention_dropout=0.0, initializer_range=0.02, use_cache=True,
                     transformers_version="4.51.0", layer_types=["full_attention", "full_attention"], rope_theta=10000)
    assert config_from_dict(published) == a
    assert isinstance(a, Qwen3Config) and "qwen3" in registered_architectures()


def test_config_round_trips_through_its_dict():
    for raw in (TINY_A, TINY_B):
        config = make_config(raw)
        assert config_from_dict(config.to_dict()) == config


@pytest.mark.parametrize("change, error, words", [
    ({"model_type": "gemma"}, UnsupportedModelError, "registered architectures"),
    ({"use_sliding_window": True, "sliding_window": 64}, UnsupportedModelError, "sliding-window"),
    ({"layer_types": ["full_attention", "sliding_attention"]}, UnsupportedModelError, "sliding-window"),
    ({"attn_logit_softcapping": 30.0}, UnsupportedModelError, "softcapping"),
    ({"partial_rotary_factor": 0.5}, UnsupportedModelError, "partial rotary"),
    ({"hidden_act": "gelu"}, UnsupportedModelError, "activation"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 4.0}}, UnsupportedModelError, "RoPE type"),
    ({"num_key_value_heads": 3}, UnsupportedModelError, "divisible"),
    ({"head_dim": 15}, UnsupportedModelError, "even head_dim"),
    ({"hidden_size": -4}, ConfigError, "hidden_size"),
    ({"vocab_size": "many"}, ConfigError, "vocab_size"),
])
def test_config_refusals_name_their_reason(change, error, words):
    with pytest.raises(error, match=words):
        config_from_dict(dict(TINY_A, **change))


def test_config_requires_eps():
    raw = dict(TINY_A)
    del raw["rms_norm_eps"]
    with pytest.raises(ConfigError, match="rms_norm_eps"):
        config_from_dict(raw)


def test_random_model_folder_is_seeded_and_complete(tmp_path):
    config = make_config(TINY_B)
    one = write_random_model(config, str(tmp_path / "one"), RandomInit(seed=3, std=0.03, norm_noise=0.1))
    two = write_random_model(config, str(tmp_path / "two"), RandomInit(seed=3, std=0.03, norm_noise=0.1))
    other = write_random_model(config, str(tmp_path / "other"), RandomInit(seed=4, std=0.03, norm_noise=0.1))
    a, b, c = (load_file(os.path.join(f, "model.safetensors")) for f in (one, two, other))
    assert set(a) == set(build_model(config).param_specs())
    assert all(torch.equal(a[k], b[k]) for k in a)
    assert not torch.equal(a["model.embed_tokens.weight"], c["model.embed_tokens.weight"])
    assert load_config(one) == config
    assert a["lm_head.weight"].shape == (384, 96) and a["model.layers.2.self_attn.q_proj.bias"].shape == (256,)
    assert abs(float(a["model.layers.0.input_layernorm.weight"].float().mean()) - 1.0) < 0.1
    assert abs(float(a["model.layers.1.mlp.up_proj.weight"].float().std()) - 0.03) < 0.003
    tied = write_random_model(make_config(TINY_A), str(tmp_path / "tied"), RandomInit(seed=1))
    assert "lm_head.weight" not in load_file(os.path.join(tied, "model.safetensors"))


def test_loader_keeps_matrices_in_compute_dtype_and_vectors_in_float32(tmp_path):
    folder = write_random_model(make_config(TINY_B), str(tmp_path / "m"), RandomInit(seed=3))
    for dtype in (torch.bfloat16, torch.float32):
        model = load_model(folder, "cpu", dtype)
        attention = model.blocks[0].mixer
        assert attention.qkv.weight.dtype == dtype and attention.qkv.weight.shape == (256 + 2 * 64, 96)
        assert attention.qkv.bias.dtype == torch.float32 and attention.q_norm_weight.dtype == torch.float32
        assert model.final_norm.weight.dtype == torch.float32
        assert model.head.weight.dtype == dtype and not model.tie_head
    stored = load_file(os.path.join(folder, "model.safetensors"))
    model = load_model(folder, "cpu", torch.bfloat16)
    fused = torch.cat([stored[f"model.layers.1.self_attn.{p}_proj.weight"] for p in "qkv"])
    assert torch.equal(model.blocks[1].mixer.qkv.weight, fused)           # stacked q, k, v; values untouched


def test_tied_head_aliases_the_embedding(tmp_path):
    folder = write_random_model(make_config(TINY_A), str(tmp_path / "m"), RandomInit(seed=3))
    model = load_model(folder, "cpu", torch.float32)
    assert model.head.weight.data_ptr() == model.embedding.weight.data_ptr()
    # an untied configuration whose file has no head is tied as well
    raw = dict(TINY_A, tie_word_embeddings=False)
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(raw, handle)
    model = load_model(folder, "cpu", torch.float32)
    assert model.head.weight.data_ptr() == model.embedding.weight.data_ptr()


def test_one_error_lists_missing_unexpected_and_misshapen_tensors(tmp_path):
    folder = write_random_model(make_config(TINY_B), str(tmp_path / "m"), RandomInit(seed=3))
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.rotary.inv_freq"] = torch.zeros(4)
    tensors["model.layers.2.self_attn.k_proj.weight"] = torch.zeros(64, 95, dtype=torch.bfloat16)
    save_file(tensors, path)
    with pytest.raises(WeightsError) as caught:
        load_model(folder, "cpu", torch.float32)
    error = caught.value
    assert error.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert error.unexpected == ["model.layers.0.self_attn.rotary.inv_freq"]
    assert [(n, tuple(f), tuple(w)) for n, f, w in error.wrong_shape] == [("model.layers.2.self_attn.k_proj.weight", (64, 95), (64, 96))]
    text = str(error)
    for word in ("missing tensors (2)", "unexpected tensors (1)", "wrong shapes (1)", "up_proj", "inv_freq", "(64, 95)"):
        assert word in text


def test_sharded_folder_is_read_through_its_index(tmp_path):
    folder = write_random_model(make_config(TINY_A), str(tmp_path / "m"), RandomInit(seed=3))
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    os.remove(os.path.join(folder, "model.safetensors"))
    names = sorted(tensors)
    shards = {"model-00001-of-00002.safetensors": names[::2], "model-00002-of-00002.safetensors": names[1::2]}
    for file_name, keys in shards.items():
        save_file({k: tensors[k] for k in keys}, os.path.join(folder, file_name))
    with open(os.path.join(folder, "model.safetensors.index.json"), "w") as handle:
        json.dump({"weight_map": {k: f for f, keys in shards.items() for k in keys}}, handle)
    model = load_model(folder, "cpu", torch.float32)
    assert torch.equal(model.embedding.weight, tensors["model.embed_tokens.weight"].float())


def test_missing_folder_parts_are_named(tmp_path):
    with pytest.raises(FileNotFoundError, match="config.json"):
        load_config(str(tmp_path))
    with open(tmp_path / "config.json", "w") as handle:
        json.dump(TINY_A, handle)
    with pytest.raises(FileNotFoundError, match="model.safetensors"):
        load_model(str(tmp_path), "cpu", torch.float32)


def test_random_model_command_writes_a_folder_that_loads_and_repeats(tmp_path):
    """bin/random_model: a named size, then the config.json it wrote: the same seed gives the same tensors."""
    import subprocess
    import sys
    from safetensors import safe_open
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    command = [sys.executable, os.path.join(root, "bin", "random_model")]
    first, second = str(tmp_path / "first"), str(tmp_path / "second")
    done = subprocess.run(command + ["--random-config", "tiny-b", "--out", first, "--seed", "3", "--norm-noise", "0.1"], capture_output=True, text=True)
    assert done.returncode == 0 and "model.safetensors" in done.stdout, done.stderr
    done = subprocess.run(command + ["--config", os.path.join(first, "config.json"), "--out", second, "--seed", "3", "--norm-noise", "0.1",
                                     "--dtype", "float32"], capture_output=True, text=True)
    assert done.returncode == 0, done.stderr
    model = load_model(first, "cpu", torch.float32)
    assert model.config.num_hidden_layers == 3 and model.config.attention_bias
    with safe_open(os.path.join(first, "model.safetensors"), "pt") as a, safe_open(os.path.join(second, "model.safetensors"), "pt") as b:
        assert sorted(a.keys()) == sorted(b.keys())
        for name in a.keys():
            assert a.get_tensor(name).dtype == torch.bfloat16 and b.get_tensor(name).dtype == torch.float32
            assert torch.equal(a.get_tensor(name), b.get_tensor(name).to(torch.bfloat16)), name
    assert os.stat(os.path.join(first, "model.safetensors")).st_mode & 0o044 == 0o044
    assert subprocess.run(command + ["--out", first], capture_output=True).returncode == 2          # neither a config nor a named size


def test_benchmark_command_takes_the_reference_name_of_its_dtype_option(capsys):
    """``--custom-dtype`` (benchmark.py:344): source and fp32 are other names of --dtype; fp16 is refused
    before anything is loaded."""
    from llmserver_amd.cli import benchmark
    with pytest.raises(SystemExit) as refused:
        benchmark.main(["--random-config", "tiny-a", "--custom-dtype", "fp16"])
    assert refused.value.code == 2
    assert "fp16" in capsys.readouterr().err
