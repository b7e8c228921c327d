"""Pins the plain implementation by what fixes it beside the reference's text: special cases
that reduce to a library routine, and invariants, each chosen so that a plausible mistake (a
wrong sign or pairing in the rotation, a norm in the wrong place, a wrong head grouping) fails."""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_qwen3 as plain

torch.manual_seed(0)
D64 = torch.float64


def tiny_tensors(config, std=0.3, seed=0):
    g = torch.Generator().manual_seed(seed)
    n_q, n_kv, d, h, i, v = (config["num_attention_heads"], config["num_key_value_heads"], plain.head_dim_of(config),
                             config["hidden_size"], config["intermediate_size"], config["vocab_size"])
    def r(*shape, scale=std):
        return scale * torch.randn(*shape, generator=g, dtype=D64)
    tensors = {"model.embed_tokens.weight": r(v, h), "model.norm.weight": 1 + r(h, scale=0.1), "lm_head.weight": r(v, h)}
    for layer in range(config["num_hidden_layers"]):
        p = f"model.layers.{layer}"
        tensors.update({
            f"{p}.input_layernorm.weight": 1 + r(h, scale=0.1), f"{p}.post_attention_layernorm.weight": 1 + r(h, scale=0.1),
            f"{p}.self_attn.q_proj.weight": r(n_q * d, h), f"{p}.self_attn.k_proj.weight": r(n_kv * d, h),
            f"{p}.self_attn.v_proj.weight": r(n_kv * d, h), f"{p}.self_attn.o_proj.weight": r(h, n_q * d),
            f"{p}.self_attn.q_norm.weight": 1 + r(d, scale=0.1), f"{p}.self_attn.k_norm.weight": 1 + r(d, scale=0.1),
            f"{p}.mlp.gate_proj.weight": r(i, h), f"{p}.mlp.up_proj.weight": r(i, h), f"{p}.mlp.down_proj.weight": r(h, i)})
    return tensors


CONFIG = dict(num_hidden_layers=2, hidden_size=24, num_attention_heads=6, num_key_value_heads=2, head_dim=8,
              intermediate_size=40, vocab_size=50, rope_theta=100.0, rms_norm_eps=1e-5)


def test_rms_norm_is_the_library_routine():
    x, w = torch.randn(5, 24, dtype=D64), torch.randn(24, dtype=D64)
    assert torch.allclose(plain.rms_norm(x, w, 1e-5), F.rms_norm(x, (24,), w, 1e-5), atol=1e-12)


def test_rms_norm_weight_is_applied_after_normalising():
    x = torch.randn(3, 8, dtype=D64)
    w = torch.arange(1.0, 9.0, dtype=D64)
    unit = plain.rms_norm(x, torch.ones(8, dtype=D64), 0.0)
    assert torch.allclose(unit.pow(2).mean(-1), torch.ones(3, dtype=D64))
    assert torch.allclose(plain.rms_norm(x, w, 0.0), unit * w)


def test_attention_without_rotation_or_mask_pressure_is_library_attention():
    q, k, v = (torch.randn(6, 9, 8, dtype=D64) for _ in range(3))
    expected = F.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True, scale=0.37)[0]
    assert torch.allclose(plain.causal_attention(q, k, v, 0.37), expected, atol=1e-12)


def test_grouped_heads_use_kv_head_h_div_g():
    """Query head h reads KV head h // G: equals library attention over repeat_interleave'd heads,
    and differs from the tiled (h % Hkv) grouping."""
    q = torch.randn(6, 7, 8, dtype=D64)
    k, v = torch.randn(2, 7, 8, dtype=D64), torch.randn(2, 7, 8, dtype=D64)
    expected = F.scaled_dot_product_attention(q[None], k.repeat_interleave(3, 0)[None], v.repeat_interleave(3, 0)[None],
                                              is_causal=True, scale=8 ** -0.5)[0]
    got = plain.causal_attention(q, k, v, 8 ** -0.5)
    assert torch.allclose(got, expected, atol=1e-12)
    tiled = F.scaled_dot_product_attention(q[None], k.repeat(3, 1, 1)[None], v.repeat(3, 1, 1)[None], is_causal=True, scale=8 ** -0.5)[0]
    assert not torch.allclose(got, tiled, atol=1e-3)


def test_one_head_one_key_returns_the_value():
    q, k, v = torch.randn(1, 1, 8, dtype=D64), torch.randn(1, 1, 8, dtype=D64), torch.randn(1, 1, 8, dtype=D64)
    assert torch.allclose(plain.causal_attention(q, k, v, 1.0), v)


def test_window_keeps_exactly_the_last_keys():
    q, k, v = (torch.randn(2, 10, 8, dtype=D64) for _ in range(3))
    full = plain.causal_attention(q, k, v, 0.5)
    assert torch.allclose(plain.causal_attention(q, k, v, 0.5, window=10), full)
    windowed = plain.causal_attention(q, k, v, 0.5, window=3)
    assert torch.allclose(windowed[:, :3], full[:, :3])
    scores = torch.einsum("hd,hkd->hk", q[:, 9], k[:, 7:10]) * 0.5      # last query over keys 7, 8, 9 only
    expected = torch.einsum("hk,hkd->hd", torch.softmax(scores, -1), v[:, 7:10])
    assert torch.allclose(windowed[:, 9], expected)


def test_rotation_is_identity_at_position_zero_and_keeps_pair_norms():
    x = torch.randn(3, 5, 8, dtype=D64)
    cos, sin = plain.rope_cos_sin(torch.zeros(5, dtype=torch.long), 8, 100.0)
    assert torch.allclose(plain.apply_rope(x, cos, sin), x)
    cos, sin = plain.rope_cos_sin(torch.arange(5), 8, 100.0)
    y = plain.apply_rope(x, cos, sin)
    assert torch.allclose(x[..., :4] ** 2 + x[..., 4:] ** 2, y[..., :4] ** 2 + y[..., 4:] ** 2)   # pairs are (i, i + d/2)
    assert not torch.allclose(x[..., 0::2] ** 2 + x[..., 1::2] ** 2, y[..., 0::2] ** 2 + y[..., 1::2] ** 2)


def test_rotation_sign_and_frequency_order():
    """x = e_0 at position p turns into (cos p, 0.., sin p at index d/2, 0..): angle of pair 0 is p * theta^0."""
    x = torch.zeros(1, 1, 8, dtype=D64)
    x[..., 0] = 1.0
    cos, sin = plain.rope_cos_sin(torch.tensor([3]), 8, 100.0)
    y = plain.apply_rope(x, cos, sin)[0, 0]
    expected = torch.zeros(8, dtype=D64)
    expected[0], expected[4] = math.cos(3.0), math.sin(3.0)
    assert torch.allclose(y, expected)
    x = torch.zeros(1, 1, 8, dtype=D64)
    x[..., 1] = 1.0                                  # pair 1 turns by p * theta^(-2/8)
    y = plain.apply_rope(x, cos, sin)[0, 0]
    angle = 3.0 * float(torch.tensor(100.0, dtype=torch.float32) ** torch.tensor(-0.25, dtype=torch.float32))
    assert abs(float(y[1]) - math.cos(angle)) < 1e-6 and abs(float(y[5]) - math.sin(angle)) < 1e-6


def test_rotated_scores_depend_on_distance_only():
    q, k = torch.randn(1, 1, 8, dtype=D64), torch.randn(1, 1, 8, dtype=D64)
    def score(pq, pk):
        cq, sq = plain.rope_cos_sin(torch.tensor([pq]), 8, 100.0, angle_dtype=angle_dtype)
        ck, sk = plain.rope_cos_sin(torch.tensor([pk]), 8, 100.0, angle_dtype=angle_dtype)
        return float((plain.apply_rope(q, cq, sq) * plain.apply_rope(k, ck, sk)).sum())
    angle_dtype = D64                                 # exact angles: the invariance is exact
    assert abs(score(7, 3) - score(107, 103)) < 1e-9
    assert abs(score(7, 3) - score(7, 4)) > 1e-6
    angle_dtype = torch.float32                       # the reference's float32 angles: exact up to their rounding
    assert abs(score(7, 3) - score(107, 103)) < 1e-4


def test_whole_model_is_invariant_to_a_shift_of_all_positions(monkeypatch):
    tensors = tiny_tensors(CONFIG)
    tokens = [3, 9, 1, 44, 17, 5, 5, 30]
    with_float32_angles = plain.forward(CONFIG, tensors, tokens)
    monkeypatch.setattr(plain, "ANGLE_DTYPE", D64)        # exact angles: the invariance is exact
    base = plain.forward(CONFIG, tensors, tokens)
    shifted = plain.forward(CONFIG, tensors, tokens, first_position=57)
    assert torch.allclose(base, shifted, atol=1e-9)
    assert torch.allclose(base, with_float32_angles, atol=1e-5)   # the reference's float32 angles differ by their rounding only


def test_swiglu_is_silu_gate_times_up():
    tensors = tiny_tensors(CONFIG)
    x = torch.randn(4, 24, dtype=D64)
    p = "model.layers.0.mlp"
    gate, up = x @ tensors[f"{p}.gate_proj.weight"].T, x @ tensors[f"{p}.up_proj.weight"].T
    expected = (gate * torch.sigmoid(gate) * up) @ tensors[f"{p}.down_proj.weight"].T
    assert torch.allclose(plain.swiglu_mlp(x, tensors, p), expected, atol=1e-12)
    swapped = (up * torch.sigmoid(up) * gate) @ tensors[f"{p}.down_proj.weight"].T
    assert not torch.allclose(plain.swiglu_mlp(x, tensors, p), swapped, atol=1e-6)


def test_model_with_silent_blocks_is_head_of_norm_of_embedding():
    tensors = tiny_tensors(CONFIG)
    for layer in range(2):
        tensors[f"model.layers.{layer}.self_attn.o_proj.weight"].zero_()
        tensors[f"model.layers.{layer}.mlp.down_proj.weight"].zero_()
    tokens = [1, 2, 3]
    h = tensors["model.embed_tokens.weight"][tokens]
    expected = F.rms_norm(h, (24,), tensors["model.norm.weight"], 1e-5) @ tensors["lm_head.weight"].T
    assert torch.allclose(plain.forward(CONFIG, tensors, tokens), expected, atol=1e-12)


def test_tied_head_uses_the_embedding_table():
    tensors = tiny_tensors(CONFIG)
    tied = dict(CONFIG, tie_word_embeddings=True)
    a = plain.forward(tied, tensors, [4, 5])
    del tensors["lm_head.weight"]
    b = plain.forward(CONFIG, tensors, [4, 5])          # no head in the file: tied as well
    assert torch.allclose(a, b)


def test_later_tokens_do_not_change_earlier_logits():
    tensors = tiny_tensors(CONFIG)
    tokens = [3, 9, 1, 44, 17, 5]
    assert torch.allclose(plain.forward(CONFIG, tensors, tokens)[:4], plain.forward(CONFIG, tensors, tokens[:4]), atol=1e-10)


def test_norm_sits_before_the_mixer_not_after():
    """Pre-norm: the mixer reads norm(h), so its update does not change when h is scaled (eps 0),
    while the residual stream carries the scale.  A norm after the mixer would fail this."""
    tensors = tiny_tensors(CONFIG)
    tensors["model.layers.0.mlp.down_proj.weight"].zero_()
    config0 = dict(CONFIG, rms_norm_eps=0.0)
    h = torch.randn(5, 24, dtype=D64)
    positions = torch.arange(5)
    out1 = plain.decoder_layer(h, tensors, 0, config0, positions)
    out2 = plain.decoder_layer(3.0 * h, tensors, 0, config0, positions)
    assert torch.allclose(out2 - 3.0 * h, out1 - h, atol=1e-9)
    assert (out1 - h).abs().max() > 1e-3


def test_q_and_k_norms_act_per_head_before_rotation():
    tensors = tiny_tensors(CONFIG)
    x = torch.randn(4, 24, dtype=D64)
    p = "model.layers.0.self_attn"
    base = plain.attention_block(x, tensors, p, CONFIG, torch.arange(4))
    scaled = dict(tensors)
    scaled[f"{p}.q_proj.weight"] = tensors[f"{p}.q_proj.weight"].clone()
    scaled[f"{p}.q_proj.weight"][:8] *= 5.0          # one head's queries five times larger: its norm removes it
    config0 = dict(CONFIG, rms_norm_eps=0.0)
    a = plain.attention_block(x, tensors, p, config0, torch.arange(4))
    b = plain.attention_block(x, scaled, p, config0, torch.arange(4))
    assert torch.allclose(a, b, atol=1e-9)
    assert base.shape == (4, 24)


# ---------------------------------------------------------------- the attention block against a construction from library routines
def library_attention_block(x, tensors, p, config, positions, weight_after_rotation=False, bias_after_norm=False, scale=None):
    """The block rebuilt from library routines only (``F.linear``, ``F.rms_norm``, ``F.scaled_dot_product_attention``
    with the library's own default scale) and an explicit rotation; the two switches build the plausible mistakes."""
    n_q, n_kv, d, eps = config["num_attention_heads"], config["num_key_value_heads"], config["head_dim"], config["rms_norm_eps"]
    seq = x.shape[0]
    angles = positions.to(torch.float32)[:, None] * (1.0 / config["rope_theta"] ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
    angles = torch.cat([angles, angles], -1).to(D64)

    def rotate(t):                       # [heads, seq, d]; pairs (i, i + d/2)
        half = d // 2
        return t * torch.cos(angles) + torch.cat([-t[..., half:], t[..., :half]], -1) * torch.sin(angles)

    def heads(name, n, norm_weight):
        bias = tensors.get(f"{p}.{name}.bias")
        y = F.linear(x, tensors[f"{p}.{name}.weight"], None if bias_after_norm else bias).view(seq, n, d).transpose(0, 1)
        if norm_weight is None:
            return y
        if weight_after_rotation:
            y = rotate(F.rms_norm(y, (d,), None, eps)) * norm_weight
        else:
            y = rotate(F.rms_norm(y, (d,), norm_weight, eps))
        if bias_after_norm and bias is not None:
            y = y + bias.view(n, 1, d)
        return y

    q = heads("q_proj", n_q, tensors[f"{p}.q_norm.weight"])
    k = heads("k_proj", n_kv, tensors[f"{p}.k_norm.weight"])
    v = heads("v_proj", n_kv, None)
    group = n_q // n_kv
    out = F.scaled_dot_product_attention(q[None], k.repeat_interleave(group, 0)[None], v.repeat_interleave(group, 0)[None],
                                         is_causal=True, scale=scale)[0]
    return F.linear(out.transpose(0, 1).reshape(seq, n_q * d), tensors[f"{p}.o_proj.weight"], tensors.get(f"{p}.o_proj.bias"))


def lopsided_norm_tensors(bias=False):
    """Norm weights far from one and different in the two halves of a head (a rotation mixes element i with element
    i + d/2, so a weight applied after the rotation gives another result), and, on request, large biases."""
    tensors = tiny_tensors(CONFIG)
    p = "model.layers.0.self_attn"
    tensors[f"{p}.q_norm.weight"] = torch.tensor([3.0, 0.2, 1.5, 0.1, 0.3, 2.5, 0.4, 4.0], dtype=D64)
    tensors[f"{p}.k_norm.weight"] = torch.tensor([0.2, 2.0, 0.3, 3.0, 2.5, 0.1, 1.8, 0.5], dtype=D64)
    if bias:
        g = torch.Generator().manual_seed(5)
        for name, rows in (("q_proj", 48), ("k_proj", 16), ("v_proj", 16), ("o_proj", 24)):
            tensors[f"{p}.{name}.bias"] = torch.randn(rows, generator=g, dtype=D64)
    return tensors, p


def test_scores_are_scaled_by_the_library_s_default_one_over_root_d():
    """``scale=None`` makes the library divide by sqrt(head_dim); the plain block is given no scale either."""
    tensors, p = lopsided_norm_tensors()
    x, positions = torch.randn(7, 24, dtype=D64), torch.arange(7)
    got = plain.attention_block(x, tensors, p, CONFIG, positions)
    assert torch.allclose(got, library_attention_block(x, tensors, p, CONFIG, positions), atol=1e-7)
    for wrong in (1.0, 1.0 / 8, 8 ** -0.25):
        assert not torch.allclose(got, library_attention_block(x, tensors, p, CONFIG, positions, scale=wrong), atol=1e-3)


def test_q_and_k_norm_weights_are_applied_before_the_rotation():
    tensors, p = lopsided_norm_tensors()
    x, positions = torch.randn(7, 24, dtype=D64), torch.arange(3, 10)       # away from position 0, where nothing turns
    got = plain.attention_block(x, tensors, p, CONFIG, positions)
    assert torch.allclose(got, library_attention_block(x, tensors, p, CONFIG, positions), atol=1e-7)
    after = library_attention_block(x, tensors, p, CONFIG, positions, weight_after_rotation=True)
    assert (got - after).abs().max() > 1e-2


def test_biases_belong_to_the_projections():
    """q, k and v biases are added by the projection, so the per-head norm sees them; the output bias is added last."""
    tensors, p = lopsided_norm_tensors(bias=True)
    x, positions = torch.randn(6, 24, dtype=D64), torch.arange(6)
    got = plain.attention_block(x, tensors, p, CONFIG, positions)
    assert torch.allclose(got, library_attention_block(x, tensors, p, CONFIG, positions), atol=1e-7)
    assert (got - library_attention_block(x, tensors, p, CONFIG, positions, bias_after_norm=True)).abs().max() > 1e-2
    without = {name: tensor for name, tensor in tensors.items() if not name.endswith(".bias")}
    silent = dict(tensors)
    silent[f"{p}.o_proj.weight"] = torch.zeros_like(tensors[f"{p}.o_proj.weight"])
    assert torch.allclose(plain.attention_block(x, silent, p, CONFIG, positions), tensors[f"{p}.o_proj.bias"].expand(6, 24))
    assert (got - plain.attention_block(x, without, p, CONFIG, positions)).abs().max() > 1e-2


ROPE_THETA_CASES = [          # (config.json keys, theta): utils/architecture.py:23-30 in the reference
    ({"rope_theta": 5.0, "rope_parameters": {"rope_theta": 7.0}}, 5.0),          # the top-level key wins
    ({"rope_parameters": {"rope_theta": 7.0}}, 7.0),
    ({"rope_scaling": {"rope_theta": 9.0}, "rope_parameters": {"rope_theta": 7.0}}, 9.0),   # rope_scaling is looked at first
    ({"rope_scaling": None, "rope_parameters": {"rope_theta": 7.0}}, 7.0),
    ({"rope_parameters": {"rope_type": "default"}}, 10000.0),
    ({}, 10000.0),
]


@pytest.mark.parametrize("keys, theta", ROPE_THETA_CASES)
def test_where_rope_theta_is_looked_up(keys, theta):
    """The plain implementation and the engine's typed configuration read the same places in the same order."""
    from llmserver_amd.config import config_from_dict
    assert plain.rope_theta_of(keys) == theta
    raw = dict(model_type="qwen3", vocab_size=50, hidden_size=24, intermediate_size=40, num_hidden_layers=1,
               num_attention_heads=3, num_key_value_heads=1, head_dim=16, rms_norm_eps=1e-5, **keys)
    assert config_from_dict(raw).rope_theta == theta


def test_inverse_cdf_sample_on_a_distribution_worked_out_by_hand():
    """The inverse CDF on a distribution worked out by hand: probabilities 0.1, 0.2, 0.3, 0.4 at temperature 1,
    and at temperature 0.5 their squares over 0.30."""
    logits = torch.log(torch.tensor([0.1, 0.2, 0.3, 0.4], dtype=torch.float64))
    assert [plain.inverse_cdf_sample(logits, 1.0, u)[0] for u in (0.0, 0.0999, 0.1001, 0.2999, 0.3001, 0.5999, 0.6001, 0.9999)] == [0, 0, 1, 1, 2, 2, 3, 3]
    edges = [0.01 / 0.30, 0.05 / 0.30, 0.14 / 0.30]
    assert [plain.inverse_cdf_sample(logits, 0.5, u)[0] for u in (edges[0] - 1e-9, edges[0] + 1e-9, edges[1] + 1e-9, edges[2] - 1e-9, edges[2] + 1e-9)] == [0, 1, 2, 2, 3]
    assert abs(plain.inverse_cdf_sample(logits, 1.0, 0.31)[1] - 0.01) < 1e-12


def test_rounded_oracle_rounds_at_the_reference_kernels_places():
    """The mode that says what a bfloat16 run may lose: a rounding that keeps everything is the exact oracle bit for bit;
    rounding to bfloat16 moves the logits by a few parts in a thousand of their size (8 bits at a dozen places a layer),
    to float32 by a few parts in ten million; and each place named in the docstrings rounds indeed (its output is
    representable in the rounded type)."""
    tensors = {name: plain.rounding_to(torch.bfloat16)(tensor) for name, tensor in tiny_tensors(CONFIG, std=0.2).items()}
    tokens = [3, 9, 1, 44, 17, 5, 30, 2, 2, 11, 49, 0]
    exact = plain.forward(CONFIG, tensors, tokens)
    assert torch.equal(plain.forward(CONFIG, tensors, tokens, r=plain.rounding_to(torch.float64)), exact)
    size = exact.abs().max(dim=-1).values
    for dtype, low, high in ((torch.bfloat16, 5e-4, 3e-2), (torch.float32, 1e-9, 2e-6)):
        lost = ((plain.forward(CONFIG, tensors, tokens, r=plain.rounding_to(dtype)) - exact).abs().max(dim=-1).values / size)
        assert low < float(lost.median()) and float(lost.max()) < high, (dtype, lost)
    r = plain.rounding_to(torch.bfloat16)
    x = r(torch.randn(5, 24, dtype=D64))

    def representable(t):
        return torch.equal(r(t), t)
    assert representable(plain.rms_norm(x, tensors["model.norm.weight"], 1e-5, r))
    assert representable(plain.swiglu_mlp(x, tensors, "model.layers.0.mlp", r))
    assert representable(plain.attention_block(x, tensors, "model.layers.0.self_attn", CONFIG, torch.arange(5), r=r))
    assert representable(plain.decoder_layer(x, tensors, 1, CONFIG, torch.arange(5), r=r))
    q = r(torch.randn(6, 5, 8, dtype=D64))
    cos, sin = plain.rope_cos_sin(torch.arange(5), 8, 100.0)
    assert representable(plain.apply_rope(q, cos, sin, r)) and not representable(plain.apply_rope(q, cos, sin))
    # q/k norms round before and after the weight: not the same numbers as one rounding at the end
    once, twice = plain.rms_norm(q, 1 + 0.3 * torch.randn(8, dtype=D64), 1e-5, r), None
    twice = plain.rms_norm(q, 1 + 0.3 * torch.randn(8, dtype=D64), 1e-5, r, rounds_before_weight=True)
    assert representable(once) and representable(twice)
