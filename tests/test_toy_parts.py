"""Generality of the parts, shown with toys that live in this file only: a mixer with state of its
own, a feed-forward that routes every token to one of several experts, another position encoding
and layers without any, layers with different windows, a layer run twice, a layer that reads
another layer's cache.
Each toy is registered as an architecture, written as a random model folder, loaded and stepped
through the framework's own step function in different cuts, without a change to the framework.
The CPU variants use the torch twins of the kernels, the GPU variants the HIP kernels."""
import dataclasses
import tempfile
from typing import ClassVar

import numpy as np
import pytest
import torch

import plain_qwen3 as plain
from helpers import BF16, check_against_rounded_oracle, random_tokens, relative_error
from llmserver_amd.cache import CacheManager
from llmserver_amd.config import ModelConfig, field, register_architecture
from llmserver_amd.engine import ModelRunner, StepEntry, load_model
from llmserver_amd.models.decoder import DecoderModel, LayerCall
from llmserver_amd.parts import (MATRIX, AttentionNames, FeedForward, GatedMLP, GatedMLPNames, GQAttention, Linear, Mixer, NoPosition,
                                 ParamSpec, PositionEncoding, PreNormBlock, RMSNorm, RotaryPosition, StateSpec, TokenEmbedding)
from llmserver_amd.weights import RandomInit, write_random_model
from torch_ops import TorchOps


# ----------------------------------------------------------------------------- a mixer with state
class RunningMeanMixer(Mixer):
    """out_t = W . mean(x_0 .. x_t).  Its state is the running sum, one vector per request."""

    def __init__(self, width):
        self.width = width
        self.weight = None

    def cache_spec(self):
        return StateSpec((self.width,), "float32")

    def param_specs(self):
        return {"mix.weight": ParamSpec((self.width, self.width), MATRIX, "normal")}

    def assign(self, name, tensor):
        self.weight = tensor

    def forward(self, x, ctx, cache):
        out = torch.empty_like(x)
        for row, (start, n, end) in enumerate(zip(ctx.h_row_start, ctx.h_row_len, ctx.h_row_ctx)):
            slot = int(ctx.h_state_slots[row])
            sums = cache.state[slot] + torch.cumsum(x[start:start + n].float(), dim=0)
            cache.state[slot] = sums[-1]
            counts = torch.arange(end - n + 1, end + 1, device=x.device, dtype=torch.float32)[:, None]
            out[start:start + n] = ((sums / counts) @ self.weight.float().t()).to(x.dtype)
        return out


# ----------------------------------------------------------------------------- a feed-forward with routing
class TopOneExperts(FeedForward):
    """out = p_e(x) * expert_e(x) for the expert e with the largest router probability p (softmax of the router's
    32-bit logits).  Every expert runs on every token and the others are masked out: wasteful, but free of host
    decisions, so a step with this feed-forward can still be captured into a graph."""

    def __init__(self, width, intermediate, n_experts):
        self.router = Linear(width, ("router",), (n_experts,), out_float32=True)
        self.experts = [GatedMLP(width, intermediate) for _ in range(n_experts)]

    def param_specs(self):
        specs = dict(self.router.param_specs())
        for index, expert in enumerate(self.experts):
            specs.update({f"experts.{index}.{name}": spec for name, spec in expert.param_specs().items()})
        return specs

    def assign(self, name, tensor):
        if name.startswith("router."):
            self.router.assign(name, tensor)
        else:
            _, index, rest = name.split(".", 2)
            self.experts[int(index)].assign(rest, tensor)

    def finalize(self):
        self.router.finalize()
        for expert in self.experts:
            expert.finalize()

    def forward(self, x, ctx):
        probabilities = torch.softmax(self.router.forward(x, ctx).float(), dim=-1)
        top, chosen = probabilities.max(dim=-1)
        out = torch.zeros_like(x, dtype=torch.float32)
        for index, expert in enumerate(self.experts):
            weight = torch.where(chosen == index, top, torch.zeros_like(top))[:, None]
            out += weight * expert.forward(x, ctx).float()
        return out.to(x.dtype)


# ----------------------------------------------------------------------------- another position encoding
class HarmonicPosition(PositionEncoding):
    """A rotate-half rotation whose pair i turns by position / (i + 1)^1.5: only the table of inverse
    frequencies differs from the framework's own encoding, the kernels take any such table."""

    def __init__(self, rotary_dim):
        self.rotary_dim = rotary_dim
        self._tables = {}

    def inverse_frequencies(self):
        return (torch.arange(1, self.rotary_dim // 2 + 1, dtype=torch.float32)) ** -1.5

    def rotary_table(self, device):
        # made once per device: a step that is being captured into a graph must not copy from the host
        if str(device) not in self._tables:
            self._tables[str(device)] = self.inverse_frequencies().to(device)
        return self._tables[str(device)]

    def cos_sin(self, ctx):
        return ctx.computed(("harmonic", id(self)), lambda: ctx.ops.rotary_table(ctx.positions, self.rotary_table(ctx.device)))


@dataclasses.dataclass(frozen=True)
class ToyConfig(ModelConfig):
    MODEL_TYPE: ClassVar[str] = "toy_parts"
    vocab_size: int = field("vocab_size", int)
    hidden_size: int = field("hidden_size", int)
    intermediate_size: int = field("intermediate_size", int)
    num_attention_heads: int = field("num_attention_heads", int)
    num_key_value_heads: int = field("num_key_value_heads", int)
    head_dim: int = field("head_dim", int)
    rms_norm_eps: float = field("rms_norm_eps", float)
    rope_theta: float = field("rope_theta", float)
    layer_kinds: object = field("layer_kinds", object)       # per block: "mean", or an attention window (0 = all keys)
    layer_order: object = field("layer_order", object)       # per call: [block, cache, writes]
    ffn_experts: object = field("ffn_experts", object, None)        # per block: 0 = dense, n = top-one of n experts
    position_kinds: object = field("position_kinds", object, None)  # per block: "rope", "harmonic" or "none"
    fused_names: bool = field("fused_names", bool, False)           # a checkpoint that stores q, k, v in one tensor, and other names
    tie_word_embeddings: bool = field("tie_word_embeddings", bool, False)

    @property
    def num_hidden_layers(self):
        return len(self.layer_kinds)


FUSED_ATTENTION = AttentionNames(qkv=("wqkv",), out="wo", q_norm="qn", k_norm="kn")
FUSED_MLP = GatedMLPNames(gate_up=("w13",), down="w2")
FUSED_BLOCK = ("attention_norm", "attention", "ffn_norm", "feed_forward")
FUSED_MODEL = ("tok_embeddings", "layers", "norm")


def build_toy(config: ToyConfig) -> DecoderModel:
    fused = config.fused_names
    attention_names, mlp_names = (FUSED_ATTENTION, FUSED_MLP) if fused else (AttentionNames(), GatedMLPNames())
    positions = {"rope": RotaryPosition(config.head_dim, config.rope_theta), "harmonic": HarmonicPosition(config.head_dim),
                 "none": NoPosition()}
    blocks = []
    for index, kind in enumerate(config.layer_kinds):
        if kind == "mean":
            mixer = RunningMeanMixer(config.hidden_size)
        else:
            position = positions[config.position_kinds[index] if config.position_kinds else "rope"]
            mixer = GQAttention(config.hidden_size, config.num_attention_heads, config.num_key_value_heads, config.head_dim,
                                position, qk_norm_eps=config.rms_norm_eps, window=kind or None, names=attention_names)
        n_experts = config.ffn_experts[index] if config.ffn_experts else 0
        ffn = TopOneExperts(config.hidden_size, config.intermediate_size, n_experts) if n_experts \
            else GatedMLP(config.hidden_size, config.intermediate_size, names=mlp_names)
        block_names = {"names": FUSED_BLOCK} if fused else {}
        blocks.append(PreNormBlock(RMSNorm(config.hidden_size, config.rms_norm_eps), mixer,
                                   RMSNorm(config.hidden_size, config.rms_norm_eps), ffn, **block_names))
    order = [LayerCall(b, c, bool(w)) for b, c, w in config.layer_order]
    head = Linear(config.hidden_size, ("output" if fused else "lm_head",), (config.vocab_size,), out_float32=True)
    model_names = {"names": FUSED_MODEL} if fused else {}
    return DecoderModel(config, TokenEmbedding(config.vocab_size, config.hidden_size), blocks,
                        RMSNorm(config.hidden_size, config.rms_norm_eps), head, config.tie_word_embeddings, order, **model_names)


register_architecture("toy_parts", ToyConfig, build_toy, replace=True)

BASE = dict(model_type="toy_parts", vocab_size=97, hidden_size=48, intermediate_size=80, num_attention_heads=4,
            num_key_value_heads=2, head_dim=16, rms_norm_eps=1e-5, rope_theta=1e4)
TOYS = {
    # attention, running mean, attention: a model whose layers have different mixers
    "state": dict(BASE, layer_kinds=[0, "mean", 0], layer_order=[[0, 0, 1], [1, 1, 1], [2, 2, 1]]),
    # windows of 9 and 20 keys beside layers that keep all keys: three cache groups
    "windows": dict(BASE, layer_kinds=[0, 9, 20, 0, 9], layer_order=[[i, i, 1] for i in range(5)]),
    # block 1 runs twice (shared weights, a cache for each run); the last call reads the cache block 0 wrote
    "order": dict(BASE, layer_kinds=[0, 0, 0], layer_order=[[0, 0, 1], [1, 1, 1], [1, 2, 1], [2, 0, 0]]),
    # a dense feed-forward, top-one of three experts, top-one of two
    "experts": dict(BASE, layer_kinds=[0, 0, 0], layer_order=[[i, i, 1] for i in range(3)], ffn_experts=[0, 3, 2]),
    # the framework's rotation, another table of frequencies, no rotation at all
    "positions": dict(BASE, layer_kinds=[0, 0, 0], layer_order=[[i, i, 1] for i in range(3)], position_kinds=["rope", "harmonic", "none"]),
    # a checkpoint with q, k and v in one tensor, gate and up in one tensor and names of its own; a window of 13 beside all keys
    "fused": dict(BASE, layer_kinds=[0, 13, 0], layer_order=[[i, i, 1] for i in range(3)], fused_names=True),
}
DISCONTINUOUS = {"experts"}       # a router's choice can flip under bfloat16 rounding: compared in float32 only


def usual_names(raw, tensors):
    """The tensors of a checkpoint with fused projections and names of its own, under the names the plain implementation
    reads: the stacked matrices are cut back into their projections."""
    if not raw.get("fused_names"):
        return tensors
    q_rows, kv_rows = raw["num_attention_heads"] * raw["head_dim"], raw["num_key_value_heads"] * raw["head_dim"]
    renamed = {"model.embed_tokens.weight": tensors["tok_embeddings.weight"], "model.norm.weight": tensors["norm.weight"],
               "lm_head.weight": tensors["output.weight"]}
    for layer in range(len(raw["layer_kinds"])):
        old, new = f"layers.{layer}", f"model.layers.{layer}"
        wqkv, w13 = tensors[f"{old}.attention.wqkv.weight"], tensors[f"{old}.feed_forward.w13.weight"]
        renamed.update({
            f"{new}.input_layernorm.weight": tensors[f"{old}.attention_norm.weight"],
            f"{new}.post_attention_layernorm.weight": tensors[f"{old}.ffn_norm.weight"],
            f"{new}.self_attn.q_proj.weight": wqkv[:q_rows], f"{new}.self_attn.k_proj.weight": wqkv[q_rows:q_rows + kv_rows],
            f"{new}.self_attn.v_proj.weight": wqkv[q_rows + kv_rows:], f"{new}.self_attn.o_proj.weight": tensors[f"{old}.attention.wo.weight"],
            f"{new}.self_attn.q_norm.weight": tensors[f"{old}.attention.qn.weight"],
            f"{new}.self_attn.k_norm.weight": tensors[f"{old}.attention.kn.weight"],
            f"{new}.mlp.gate_proj.weight": w13[:raw["intermediate_size"]], f"{new}.mlp.up_proj.weight": w13[raw["intermediate_size"]:],
            f"{new}.mlp.down_proj.weight": tensors[f"{old}.feed_forward.w2.weight"]})
    return renamed


def plain_toy(raw, tensors, tokens, r=plain.exact):
    """The toy models over a whole sequence, from the plain implementation's functions; with a rounding ``r`` the
    intermediate results round where the plain implementation's functions round theirs (and the toys' own parts after
    each of their products), which says what a bfloat16 run of the toy may lose."""
    tensors = usual_names(raw, tensors)
    config = dict(raw, num_hidden_layers=len(raw["layer_kinds"]))
    ids = torch.as_tensor(tokens)
    positions = torch.arange(len(tokens))
    h = tensors["model.embed_tokens.weight"][ids]
    eps = raw["rms_norm_eps"]
    stored, cache_owner = {}, {}
    for block, cache, writes in raw["layer_order"]:
        prefix = f"model.layers.{block}"
        kind = raw["layer_kinds"][block]
        normed = plain.rms_norm(h, tensors[f"{prefix}.input_layernorm.weight"], eps, r)
        if kind == "mean":
            counts = torch.arange(1, len(tokens) + 1, dtype=h.dtype)[:, None]
            mixed = r((torch.cumsum(normed, 0) / counts) @ tensors[f"{prefix}.self_attn.mix.weight"].T)
        else:
            slot = f"cache{cache}"
            local = {}
            position_kind = raw["position_kinds"][block] if raw.get("position_kinds") else "rope"
            cos_sin = None
            if position_kind != "rope":
                pairs = raw["head_dim"] // 2
                rates = torch.arange(1, pairs + 1, dtype=h.dtype) ** -1.5 if position_kind == "harmonic" else torch.zeros(pairs, dtype=h.dtype)
                angles = positions.to(h.dtype)[:, None] * torch.cat([rates, rates])[None, :]
                cos_sin = (torch.cos(angles), torch.sin(angles))
            mixed = plain.attention_block(normed, tensors, f"{prefix}.self_attn", config, positions, kind or None,
                                          kv_store=local if writes else stored, kv_from=None if writes else slot, cos_sin=cos_sin, r=r)
            if writes:
                stored[slot] = local[f"{prefix}.self_attn"]
        h = r(h + mixed)
        normed = plain.rms_norm(h, tensors[f"{prefix}.post_attention_layernorm.weight"], eps, r)
        n_experts = raw["ffn_experts"][block] if raw.get("ffn_experts") else 0
        if n_experts:
            probabilities = torch.softmax(normed @ tensors[f"{prefix}.mlp.router.weight"].T, dim=-1)
            top, chosen = probabilities.max(dim=-1)
            update = torch.zeros_like(h)
            for expert in range(n_experts):
                rows = chosen == expert
                update[rows] = r(top[rows, None] * plain.swiglu_mlp(normed[rows], tensors, f"{prefix}.mlp.experts.{expert}", r))
            h = r(h + update)
        else:
            h = r(h + plain.swiglu_mlp(normed, tensors, f"{prefix}.mlp", r))
    return plain.rms_norm(h, tensors["model.norm.weight"], eps, r) @ tensors["lm_head.weight"].T


def run_toy(name, device, dtype, ops, tol=None):
    """``tol``: the largest difference allowed (float32); None: a bfloat16 run, held against what the toy's plain
    implementation loses when it rounds to bfloat16 (helpers.check_against_rounded_oracle)."""
    raw = TOYS[name]
    from llmserver_amd.config import config_from_dict
    folder = tempfile.mkdtemp(prefix=f"llmserver_amd_toy_{name}_")
    write_random_model(config_from_dict(dict(raw)), folder, RandomInit(seed=9, std=0.08, norm_noise=0.1))
    model = load_model(folder, device, dtype)
    _, tensors = plain.read_folder(folder)
    page = 4
    cache = CacheManager(model.cache_specs(), page, 36, num_state_slots=2, device=device, dtype=model.dtype)
    if name == "windows":
        assert sorted(str(g.spec.window) for g in cache.groups) == ["20", "9", "None"]
    if name == "fused":
        assert sorted(str(g.spec.window) for g in cache.groups) == ["13", "None"]
        assert "layers.1.attention.wqkv.weight" in tensors and model.blocks[1].mixer.qkv.weight.shape == (8 * 16, 48)
    if name == "state":
        assert cache.state_specs and not cache.prefix_caching_possible
    runner = ModelRunner(model, cache, ops)
    sequences = {"x": random_tokens(97, 75, 1), "y": random_tokens(97, 52, 2)}
    expected = {rid: plain_toy(raw, tensors, tokens) for rid, tokens in sequences.items()}
    lost = [] if tol is not None else [relative_error(row, exact) for rid, tokens in sequences.items()
                                       for row, exact in zip(plain_toy(raw, tensors, tokens, BF16).numpy(), expected[rid].numpy())]
    errors = []
    cuts = {"x": [0, 30, 31, 33, 60, 61, 62, 75], "y": [0, 2, 27, 28, 29, 50, 51, 52]}
    got = {rid: [] for rid in sequences}
    for rid in sequences:
        cache.open(rid)
    for turn in range(7):                      # both requests in every step: portions beside single tokens
        entries = []
        for rid, tokens in sequences.items():
            a, b = cuts[rid][turn], cuts[rid][turn + 1]
            entries.append(StepEntry(rid, tokens[a:b], list(range(b - a))))
        logits = runner.step(entries).double().cpu()
        row = 0
        for entry in entries:
            got[entry.request_id].append(logits[row:row + len(entry.tokens)])
            row += len(entry.tokens)
        cache.check_invariants()
    if name == "windows":
        tables = cache.record("x").tables
        window9 = next(g.index for g in cache.groups if g.spec.window == 9)
        assert tables[window9][:15] == [-1] * 15 and all(p >= 0 for p in tables[window9][17:])   # pages the window passed are gone
    for rid in sequences:
        if tol is not None:
            error = float((torch.cat(got[rid]) - expected[rid]).abs().max())
            assert error < tol, (name, rid, error)
        errors += [relative_error(row, exact) for row, exact in zip(torch.cat(got[rid]).numpy(), expected[rid].numpy())]
        cache.close(rid)
    cache.check_invariants()
    assert all(g.pool.num_available == g.pool.num_pages for g in cache.groups)
    # the same request again, whole, through pages that were used before
    cache.open("again")
    whole = runner.step([StepEntry("again", sequences["x"], list(range(75)))]).double().cpu()
    if tol is not None:
        assert float((whole - expected["x"]).abs().max()) < tol
    else:
        errors += [relative_error(row, exact) for row, exact in zip(whole.numpy(), expected["x"].numpy())]
        check_against_rounded_oracle(errors, lost, f"toy {name}")
    cache.close("again")


@pytest.mark.parametrize("name", sorted(TOYS))
def test_toy_on_cpu(name):
    run_toy(name, "cpu", "float32", TorchOps(), 5e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype, tol", [("float32", 5e-5), ("bfloat16", None)])
@pytest.mark.parametrize("name", sorted(TOYS))
def test_toy_on_gpu(name, dtype, tol):
    print(f"toy {name} {dtype}", flush=True)
    if name in DISCONTINUOUS and dtype != "float32":
        pytest.skip("a router's choice can flip under bfloat16 rounding; this toy is compared in float32")
    from llmserver_amd.kernels import default_ops
    run_toy(name, "cuda", dtype, default_ops(), tol)
