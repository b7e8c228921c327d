"""Each part alone on the GPU against the plain implementation's function for it."""
import pytest
import torch

import plain_qwen3 as plain
from helpers import BF16, check_against_rounded_oracle, relative_error
from llmserver_amd.cache import CacheManager
from llmserver_amd.engine.batch import Staging, StepContext
from llmserver_amd.models.decoder import LayerCall
from llmserver_amd.parts import GatedMLP, GQAttention, Linear, PreNormBlock, RMSNorm, RotaryPosition, TokenEmbedding

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = {torch.float32: 3e-5}


def held(got, exact, rounded, dtype, what, slack=1):
    """float32: within a fixed distance of the plain function's result.  bfloat16: row by row in units of the row's
    largest number, against what the plain function loses when it rounds to bfloat16 where the reference's kernels
    round (``rounded`` is its result then)."""
    got, exact = got.double().cpu(), exact.double()
    if dtype == torch.float32:
        assert float((got - exact).abs().max()) < TOL[dtype] * slack, what
        return
    check_against_rounded_oracle([relative_error(g, e) for g, e in zip(got.numpy(), exact.numpy())],
                                 [relative_error(r, e) for r, e in zip(rounded.double().numpy(), exact.numpy())], what)
CONFIG = dict(hidden_size=72, num_attention_heads=6, num_key_value_heads=2, head_dim=48, intermediate_size=100,
              rope_theta=5e4, rms_norm_eps=3e-6)


def context(dtype, lens, starts):
    from llmserver_amd.kernels import default_ops
    ctx = StepContext(default_ops(), DEV, dtype, Staging(DEV))
    positions = [p for s, n in zip(starts, lens) for p in range(s, s + n)]
    token_row = [r for r, n in enumerate(lens) for _ in range(n)]
    row_start = [sum(lens[:r]) for r in range(len(lens))]
    return ctx, positions, token_row, row_start


def fill(part, tensors, dtype):
    for name, spec in part.param_specs().items():
        kind = dtype if spec.role == "matrix" else torch.float32
        part.assign(name, tensors[name].to(device=DEV, dtype=kind).contiguous())
    part.finalize()


def weights(specs, seed):
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, spec in specs.items():
        x = torch.randn(spec.shape, generator=g)
        out[name] = (1 + 0.1 * x if spec.init == "norm" else 0.2 * x).to(torch.bfloat16).double()
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_mlp_embedding_linear(dtype):
    print(f"parts norm/mlp/embedding/linear {dtype}", flush=True)
    ctx, *_ = context(dtype, [9], [0])
    inputs = torch.Generator().manual_seed(21)              # the same inputs whatever ran before
    x = torch.randn(9, 72, generator=inputs).to(torch.bfloat16).double()
    delta = torch.randn(9, 72, generator=inputs).to(torch.bfloat16).double()
    norm = RMSNorm(72, 3e-6)
    w = weights(norm.param_specs(), 1)
    fill(norm, w, dtype)
    resid = x.to(device=DEV, dtype=dtype)
    got = norm.add_norm(resid, delta.to(device=DEV, dtype=dtype), ctx)
    held(got, plain.rms_norm(x + delta, w["weight"], 3e-6), plain.rms_norm(BF16(x + delta), w["weight"], 3e-6, BF16), dtype, "norm of the sum")
    held(resid, x + delta, BF16(x + delta), dtype, "the sum, stored back")

    mlp = GatedMLP(72, 100)
    w = weights(mlp.param_specs(), 2)
    fill(mlp, w, dtype)
    # (nine rows at a time, the few-row kernels' case; eight draws of them, so that the spread of the errors shows)
    draws = [torch.randn(9, 72, generator=inputs).to(torch.bfloat16).double() for _ in range(8)]
    got = torch.cat([mlp.forward(draw.to(device=DEV, dtype=dtype), ctx) for draw in draws])
    named, many = {f"m.{k}": v for k, v in w.items()}, torch.cat(draws)
    held(got, plain.swiglu_mlp(many, named, "m"), plain.swiglu_mlp(many, named, "m", BF16), dtype, "gated feed-forward", slack=10)

    table = TokenEmbedding(301, 72)
    w = weights(table.param_specs(), 3)
    fill(table, w, dtype)
    ids = torch.tensor([300, 0, 7], dtype=torch.int32, device=DEV)
    assert torch.equal(table.forward(ids, ctx).double().cpu(), w["weight"][[300, 0, 7]].to(dtype).double())

    linear = Linear(72, ("a", "b"), (10, 30), bias=True, out_float32=True)
    w = weights(linear.param_specs(), 4)
    fill(linear, w, dtype)
    got = linear.forward(x.to(device=DEV, dtype=dtype), ctx)
    expected = torch.cat([x @ w["a.weight"].T + w["a.bias"], x @ w["b.weight"].T + w["b.bias"]], dim=1)
    assert got.dtype == torch.float32
    held(got, expected, BF16(expected), dtype, "stacked projection with biases, 32-bit result", slack=10)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("bias", [False, True])
def test_attention_part_and_block(dtype, bias):
    """One request, fed in three steps (a portion, a decoded token, another portion) through the
    attention part and through a whole block, against the plain functions on the whole sequence."""
    print(f"parts attention/block {dtype} bias {bias}", flush=True)
    page = 12
    attention = GQAttention(72, 6, 2, 48, RotaryPosition(48, 5e4), qk_norm_eps=3e-6, bias=bias)
    block = PreNormBlock(RMSNorm(72, 3e-6), attention, RMSNorm(72, 3e-6), GatedMLP(72, 100))
    w = weights(block.param_specs(), 5)
    fill(block, w, dtype)
    named = {f"model.layers.0.{k}": v for k, v in w.items()}
    config = dict(CONFIG, num_hidden_layers=1)
    x = torch.randn(30, 72, generator=torch.Generator().manual_seed(22)).to(torch.bfloat16).double()
    positions = torch.arange(30)
    expected_attention = plain.attention_block(x, named, "model.layers.0.self_attn", config, positions)
    expected_block = plain.decoder_layer(x, named, 0, config, positions)
    rounded = {"attention": plain.attention_block(x, named, "model.layers.0.self_attn", config, positions, r=BF16),
               "block": plain.decoder_layer(x, named, 0, config, positions, r=BF16)}
    for what in ("attention", "block"):
        cache = CacheManager({0: attention.cache_spec()}, page, 4, device=DEV, dtype=dtype)
        cache.open("r")
        outs = []
        for start, end in ((0, 13), (13, 14), (14, 30)):
            n = end - start
            cache.ensure("r", end)
            ctx, pos, token_row, row_start = context(dtype, [n], [start])
            ctx.page_size = page                          # as the step function says it: the plan asks the kernels with it
            table = torch.tensor([cache.record("r").tables[0]], dtype=torch.int32).numpy()
            ctx.fill([0] * n, pos, token_row, row_start, [n], [end], [], [table], None, ["r"])
            attention.prepare(ctx)
            ctx.upload()
            view = cache.view(LayerCall(0, 0))
            chunk = x[start:end].to(device=DEV, dtype=dtype)
            if what == "attention":
                outs.append(attention.forward(chunk, ctx, view).double().cpu())
            else:
                resid, delta = block.forward(chunk.clone(), None, ctx, view)
                outs.append((resid.double() + delta.double()).cpu())
            cache.advance("r", end)
        got = torch.cat(outs)
        expected = expected_attention if what == "attention" else expected_block
        held(got, expected, rounded[what], dtype, f"{what} in three steps", slack=4 if what == "attention" else 10)


def test_block_without_fused_stream_updates():
    """The same block with every residual sum and norm as a kernel of its own (the few-row projections
    otherwise fold them into their epilogues)."""
    from llmserver_amd.kernels import default_ops
    ops = default_ops()
    ops.fuse_stream_updates = False
    try:
        test_attention_part_and_block(torch.bfloat16, True)
        test_attention_part_and_block(torch.bfloat16, False)
    finally:
        ops.fuse_stream_updates = True
