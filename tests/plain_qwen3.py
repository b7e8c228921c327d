"""A plain, slow implementation of the Qwen3 dense decoder: whole sequences, no cache, one
function for each part, written from the reference's formulas.  It shares no code with the
engine (it reads config.json and the safetensors file itself) and is the oracle of the tests.
Every function cites the lines of the reference it follows.  Arithmetic is float64 by default so
that the oracle's own rounding is far below the tolerances used against it.

Every function also takes ``r``, a rounding of intermediate results that stands where the reference's
bfloat16 kernels round theirs (:func:`rounding_to`); with it the same formulas say how far a faultless
bfloat16 run of this model, on these tokens, lies from the exact result.  That distance, and not a
constant, is what a bfloat16 engine's error is measured against.  ``exact`` (the default) rounds nothing.
"""
from __future__ import annotations

import json
import math
import os

import torch
from safetensors import safe_open


def exact(x):
    return x


def rounding_to(dtype):
    """``x -> x`` rounded to ``dtype`` and widened back to the type it came in."""
    return lambda x: x.to(dtype).to(x.dtype)


def read_folder(folder, dtype=torch.float64):
    """config.json as a dict and every tensor of model.safetensors, widened to ``dtype``."""
    with open(os.path.join(folder, "config.json")) as handle:
        config = json.load(handle)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as handle:
        for name in handle.keys():
            tensors[name] = handle.get_tensor(name).to(dtype)
    return config, tensors


def head_dim_of(config):
    """utils/architecture.py:88"""
    return config.get("head_dim") or config["hidden_size"] // config["num_attention_heads"]


def rope_theta_of(config):
    """utils/architecture.py:23-30"""
    parameters = config.get("rope_scaling") or config.get("rope_parameters") or {}
    theta = config.get("rope_theta")
    return parameters.get("rope_theta", 10000.0) if theta is None else theta


def rms_norm(x, weight, eps, r=exact, rounds_before_weight=False):
    """y = x * rsqrt(mean(x^2, last dim) + eps) * w  (utils/layers.py:133-138).

    Rounded once where the reference's kernel of the residual sum and the norm rounds (utils/fused_ops.py:78), or, for
    the per-head norms of q and k, before and after the weight (``rounds_before_weight``: utils/fused_ops.py:110-111,
    as utils/layers.py:137-138 does)."""
    variance = x.pow(2).mean(dim=-1, keepdim=True)
    normalized = x * torch.rsqrt(variance + eps)
    return r(weight * r(normalized)) if rounds_before_weight else r(weight * normalized)


def inverse_frequencies(head_dim, theta, dtype=torch.float64):
    """inv_freq_i = 1 / theta^(2i/d), i = 0..d/2-1  (utils/layers.py:145,158).

    The reference evaluates this in float32; the float32 values are kept so that the oracle's
    angles are the ones the formula defines at the reference's precision of the table."""
    indices = torch.arange(0, head_dim, 2, dtype=torch.long)
    table = 1.0 / (theta ** (indices.to(torch.float32) / head_dim))
    return table.to(dtype)


ANGLE_DTYPE = torch.float32     # precision of pos * inv_freq, as in the reference; tests of exact invariants set float64


def rope_cos_sin(positions, head_dim, theta, dtype=torch.float64, angle_dtype=None):
    """angles = pos * inv_freq, duplicated over both halves  (utils/layers.py:160-164).

    The reference forms the product in float32 (line 160: ``pos_ids.to(torch.float32) * inv_freq``), and a
    float32 angle of a few thousand radians is up to 2e-4 away from the exact product: that rounding is
    part of the formula, so it is kept; cosine and sine of that angle are then taken in ``dtype``.
    ``angle_dtype=torch.float64`` gives the exact product (for invariants that hold only without that rounding)."""
    angle_dtype = angle_dtype or ANGLE_DTYPE
    frequencies = (positions.to(angle_dtype).unsqueeze(-1) * inverse_frequencies(head_dim, theta, angle_dtype).to(positions.device)).to(dtype)
    angles = torch.cat([frequencies, frequencies], dim=-1)
    return torch.cos(angles), torch.sin(angles)


def rotate_half(x):
    """cat(-x[d/2:], x[:d/2])  (utils/layers.py:166-170)."""
    half = x.shape[-1] // 2
    return torch.cat([-x[..., half:], x[..., :half]], dim=-1)


def apply_rope(x, cos, sin, r=exact):
    """x * cos + rotate_half(x) * sin; x [heads, seq, d], cos/sin [seq, d]  (utils/layers.py:172-177).

    Rounding: cosine and sine are held in the activations' type (utils/layers.py:164), ``x * cos`` rounds, and the sum
    with the other half's product rounds once more (utils/fused_ops.py:116-119)."""
    cos, sin = r(cos), r(sin)
    return r(r(x * cos.unsqueeze(0)) + rotate_half(x) * sin.unsqueeze(0))


def causal_attention(q, k, v, scale, window=None, r=exact):
    """q [Hq, S, d], k/v [Hkv, S, d] -> [Hq, S, d].

    Rounding: scores and softmax stay wide, the probabilities round before they meet the values
    (utils/attention.py:197, utils/paged_attention.py:212), and the result rounds as every product's does.

    KV heads repeated per group, scores scaled, causal additive mask, softmax, times V
    (utils/attention.py:188-198).  ``window`` (not in the reference, which refuses
    sliding windows at utils/architecture.py:72-76) keeps for query p the keys
    p-window+1 .. p; None keeps all."""
    n_q, seq, _ = q.shape
    group = n_q // k.shape[0]
    k = torch.repeat_interleave(k, repeats=group, dim=0)
    v = torch.repeat_interleave(v, repeats=group, dim=0)
    scores = torch.matmul(q, k.transpose(-1, -2)) * scale
    place = torch.arange(seq, device=q.device)
    hidden = place[None, :] > place[:, None]
    if window is not None:
        hidden = hidden | (place[None, :] <= place[:, None] - window)
    scores = scores.masked_fill(hidden.unsqueeze(0), float("-inf"))
    return r(torch.matmul(r(torch.softmax(scores, dim=-1)), v))


def attention_block(x, tensors, prefix, config, positions, window=None, kv_store=None, kv_from=None, cos_sin=None, r=exact):
    """Projections, per-head q/k norm before the rotation, rotation, attention, output projection
    (utils/attention.py:119-128, 155-159, 299-300).

    ``kv_store`` (a dict) receives this layer's rotated keys and values under ``prefix``;
    ``kv_from`` names a prefix whose stored keys and values are used instead of this layer's own
    (the tests' toy arrangement in which one layer reads another layer's cache).  ``cos_sin`` replaces the
    rotation's cosines and sines (the tests' toy position encodings).  A projection rounds once, after its bias."""
    n_q, n_kv, d = config["num_attention_heads"], config["num_key_value_heads"], head_dim_of(config)
    seq = x.shape[0]

    def project(name):
        y = x @ tensors[f"{prefix}.{name}.weight"].T
        bias = tensors.get(f"{prefix}.{name}.bias")
        return r(y if bias is None else y + bias)

    q = project("q_proj").view(seq, n_q, d).permute(1, 0, 2)
    k = project("k_proj").view(seq, n_kv, d).permute(1, 0, 2)
    v = project("v_proj").view(seq, n_kv, d).permute(1, 0, 2)
    q = rms_norm(q, tensors[f"{prefix}.q_norm.weight"], config["rms_norm_eps"], r, rounds_before_weight=True)
    k = rms_norm(k, tensors[f"{prefix}.k_norm.weight"], config["rms_norm_eps"], r, rounds_before_weight=True)
    cos, sin = cos_sin if cos_sin is not None else rope_cos_sin(positions, d, rope_theta_of(config), x.dtype)
    q, k = apply_rope(q, cos, sin, r), apply_rope(k, cos, sin, r)
    if kv_store is not None:
        if kv_from is not None:
            k, v = kv_store[kv_from]
        else:
            kv_store[prefix] = (k, v)
    out = causal_attention(q, k, v, d ** -0.5, window, r)        # utils/architecture.py:105
    out = out.permute(1, 0, 2).reshape(seq, n_q * d)
    y = out @ tensors[f"{prefix}.o_proj.weight"].T
    bias = tensors.get(f"{prefix}.o_proj.bias")
    return r(y if bias is None else y + bias)


def swiglu_mlp(x, tensors, prefix, r=exact):
    """down(silu(gate(x)) * up(x))  (utils/layers.py:210-218).

    Rounding: each product once; SiLU before it meets ``up``, and their product (utils/fused_ops.py:87-88)."""
    gate = r(x @ tensors[f"{prefix}.gate_proj.weight"].T)
    up = r(x @ tensors[f"{prefix}.up_proj.weight"].T)
    return r(r(r(torch.nn.functional.silu(gate)) * up) @ tensors[f"{prefix}.down_proj.weight"].T)


def decoder_layer(h, tensors, index, config, positions, window=None, r=exact):
    """h += attn(norm_in(h)); h += mlp(norm_post(h))  (utils/model.py:15-35).

    Rounding: the residual stream rounds after every sum (utils/fused_ops.py:73 of the sum-and-norm kernel: "round the
    residual stream like the unfused add"), and the norm is taken of the rounded stream."""
    prefix = f"model.layers.{index}"
    eps = config["rms_norm_eps"]
    h = r(h + attention_block(rms_norm(h, tensors[f"{prefix}.input_layernorm.weight"], eps, r), tensors,
                              f"{prefix}.self_attn", config, positions, window, r=r))
    return r(h + swiglu_mlp(rms_norm(h, tensors[f"{prefix}.post_attention_layernorm.weight"], eps, r), tensors, f"{prefix}.mlp", r))


def forward(config, tensors, token_ids, windows=None, layer_order=None, first_position=0, r=exact, places=None):
    """Logits ``[seq, vocab]`` at every position of one whole sequence
    (utils/model.py:109-158 without cache; tied head rule
    utils/model_loader.py:56-59).

    ``windows`` (per layer) and ``layer_order`` (which layer runs when) serve the tests' toy
    arrangements; ``first_position`` shifts all positions.  With a rounding ``r`` everything up to the last norm
    rounds as the reference's bfloat16 run does; the logits themselves stay wide (an engine hands out 32-bit logits,
    so the rounding of the head's result is not part of what it may lose).  ``places``: the positions whose logits are
    wanted (all of them if None; a vocabulary of 150,000 makes the others expensive).  Runs where the tensors live."""
    device = tensors["model.embed_tokens.weight"].device
    ids = torch.as_tensor(token_ids, dtype=torch.long, device=device)
    positions = torch.arange(len(ids), device=device) + first_position
    h = tensors["model.embed_tokens.weight"][ids]
    order = layer_order if layer_order is not None else range(config["num_hidden_layers"])
    for index in order:
        h = decoder_layer(h, tensors, index, config, positions, None if windows is None else windows[index], r)
    if places is not None:
        h = h[torch.as_tensor(places, dtype=torch.long, device=device)]
    h = rms_norm(h, tensors["model.norm.weight"], config["rms_norm_eps"], r)
    head = tensors["model.embed_tokens.weight"] if config.get("tie_word_embeddings") or "lm_head.weight" not in tensors \
        else tensors["lm_head.weight"]
    return h @ head.T


def greedy_generate(config, tensors, prompt, new_tokens):
    """Argmax continuation, recomputing the whole sequence each step (utils/engine.py:295-297)."""
    tokens = list(prompt)
    for _ in range(new_tokens):
        tokens.append(int(torch.argmax(forward(config, tensors, tokens)[-1])))
    return tokens[len(prompt):]


def inverse_cdf_sample(logits, temperature, uniform):
    """The token that ``uniform`` in [0, 1) picks from softmax(logits / temperature): the first token whose cumulative
    probability exceeds it; and how far ``uniform`` lies from the nearest edge between two tokens.  (Not in the
    reference, whose engine takes the argmax, utils/engine.py:295-297: this is the definition the engine's temperature
    sampling is held to.)"""
    probabilities = torch.softmax(torch.as_tensor(logits, dtype=torch.float64) / temperature, dim=-1)
    cumulative = torch.cumsum(probabilities, dim=-1)
    token = int(torch.searchsorted(cumulative, torch.tensor(uniform, dtype=torch.float64), right=True).clamp(max=len(cumulative) - 1))
    return token, float((cumulative - uniform).abs().min())
