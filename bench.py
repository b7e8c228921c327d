"""Decode and prefill throughput of the engine on one MI355X, with random weights.

    python bench.py --gpus 1 --steps K --warmup W

Default workload: the Qwen3-8B-sized configuration (36 layers, hidden 4096, 32 query heads, 8 KV
heads, head size 128, intermediate 12288, vocabulary 151936, untied head), bfloat16, a batch of 8
requests decoding at a context of 4,096 tokens.  A "step" is one decode step of the whole batch
through ``Engine.step()``: the scheduler plans it, the batch is laid out, the model runs against the
paged cache, tokens are sampled greedily and every request moves on.  Prints ONE JSON line: ``value``
is decoded tokens per second; ``prefill`` times one engine step that takes a 2,048-token prompt from
its arrival to its first token; ``roofline`` relates the bytes a decode step has to read (every
weight once, plus the cache of the live requests) to the published HBM bandwidth; ``points`` holds
batch 1 and 64 of the same model (tokens per second, with the step's milliseconds and its share of
the HBM peak beside them), prompts of 512, 8,192 and 16,384 tokens, a prompt of which all but the last 128 tokens lie in
the cache already (8,064 of them: the next turn of a conversation), four requests at a context of 16,384 and eight at
32,768, the baseline's own decode workload (prompts of 2,048 tokens decoded to 4,096, every step timed, at batch 1, 8
and 64) and, unless ``--no-extra-points``, the two other workloads the baseline
names: 64 mixed requests with a shared prefix on Qwen3-1.7B sizes, and batch 16 behind 8,192 tokens
on Qwen3-32B sizes.  Token ids are seeded uniform random numbers (synthetic data), weights seeded normal.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}
MODEL = "qwen3-8b"


def log(*args):
    print(*args, file=sys.stderr, flush=True)


def decode_step_bytes(model, batch, context):
    """What a decoding step of ``batch`` rows at ``context`` tokens has to read: every weight it uses once and the
    cache of its rows, summed over what the model's parts declare (no formula of an architecture stands here)."""
    from llmserver_amd.engine.cost import StepRow, step_bytes
    return step_bytes(model, [StepRow(1, context)] * batch, model.dtype)


def prefill_flops(model, tokens):
    """Floating-point operations of the step that takes a prompt of ``tokens`` tokens to its first token."""
    from llmserver_amd.engine.cost import StepRow, step_flops
    return step_flops(model, [StepRow(tokens, tokens, wanted=1)])


def random_model(name, layers, dtype, seed=0):
    from llmserver_amd.config import config_from_dict, named_size
    from llmserver_amd.kernels import default_ops
    from llmserver_amd.weights import RandomInit, random_model_on_device
    raw = named_size(name)
    full = raw["num_hidden_layers"]
    raw["num_hidden_layers"] = min(full, layers) if layers else full
    config = config_from_dict(raw)
    default_ops().preload([config.head_dim], dtype)
    log(f"[bench] {name}: drawing random weights")
    model = random_model_on_device(config, "cuda:0", dtype, RandomInit(seed=seed, std=0.02))
    model.name = f"{name}-random"
    log(f"[bench] {name}: a decoding step of one row reads {decode_step_bytes(model, 1, 0) / 1e9:.2f} GB of weights")
    return model, config, full


def decode_through_engine(model, page_size, batch, context, steps, warmup, seed=0):
    """Seconds for exactly ``steps`` decoding steps of ``batch`` requests through ``Engine.step()``, the last of which
    ends at a context of ``context`` tokens.  The requests' prompts are prefilled by the engine itself first."""
    import torch

    from llmserver_amd.engine import Engine, RequestStatus
    prompt_tokens = context - steps - warmup
    pages = batch * (-(-(context + 8) // page_size)) + 16
    engine = Engine(model, None, max_new_tokens=steps + warmup + 8, max_batch_size=batch, max_num_batched_tokens=max(4096, batch * page_size),
                    kv_cache_num_blocks=pages, kv_cache_block_size=page_size, stream_text=False, max_completed_requests=0,
                    ignore_eos=True, enable_prefix_caching=True)
    generator = torch.Generator().manual_seed(seed)
    vocab = model.config.vocab_size
    prompts = [torch.randint(0, vocab, (prompt_tokens,), generator=generator).tolist() for _ in range(batch)]
    # Every prompt goes through the engine once on its own, which leaves its complete pages in the cache; the requests
    # that are timed then find them, compute the last few tokens of their prompts in one common step, and decode in step.
    for prompt in prompts:
        engine.add_request(None, prompt_token_ids=prompt, max_new_tokens=1)
        while engine.step():
            pass
    requests = [engine.add_request(None, prompt_token_ids=prompt) for prompt in prompts]
    engine.step()
    assert all(request.status == RequestStatus.DECODING for request in requests), "the prompts' pages were not found in the cache"
    produced = len(requests[0].generated_token_ids)
    assert produced == 1 and all(len(request.generated_token_ids) == produced for request in requests)

    def run(count):
        # The last of these steps starts nothing ahead of time: what is timed is exactly these steps' work.
        for index in range(count):
            engine.launch_ahead = index + 1 < count
            engine.step()
        torch.cuda.synchronize()

    run(warmup + 1 - produced)                          # the step that finished the prompts gave the first token
    start = time.perf_counter()
    run(steps)
    elapsed = time.perf_counter() - start
    assert all(len(request.generated_token_ids) == warmup + 1 + steps for request in requests)
    assert all(request.sequence_length == context + 1 for request in requests)       # the last step ran at `context` tokens
    profile = dict(engine.step_profile)
    for request in requests:
        engine.cancel_request(request.request_id)
    del engine
    torch.cuda.empty_cache()
    return elapsed, profile


def prefill_through_engine(model, page_size, tokens, repeats=3, seed=1):
    """Seconds of the one engine step that takes a prompt of ``tokens`` tokens to its first token (best of ``repeats``)."""
    import torch

    from llmserver_amd.engine import Engine
    engine = Engine(model, None, max_new_tokens=1, max_batch_size=1, max_num_batched_tokens=tokens,
                    kv_cache_num_blocks=-(-tokens // page_size) + 8, kv_cache_block_size=page_size, stream_text=False,
                    max_completed_requests=0, ignore_eos=True, enable_prefix_caching=False)
    generator = torch.Generator().manual_seed(seed)
    best = float("inf")
    for attempt in range(repeats + 1):
        request = engine.add_request(None, prompt_token_ids=torch.randint(0, model.config.vocab_size, (tokens,), generator=generator).tolist())
        torch.cuda.synchronize()
        start = time.perf_counter()
        more = engine.step()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - start
        assert not more and len(request.generated_token_ids) == 1
        if attempt:
            best = min(best, elapsed)
    del engine
    torch.cuda.empty_cache()
    return best


def turn_through_engine(model, page_size, cached, fresh, repeats=3, seed=2):
    """Seconds of the one engine step that takes a prompt whose first ``cached`` tokens lie in the cache already (an
    earlier request left them there) and whose last ``fresh`` tokens are new to its first token: the next turn of a
    conversation.  Best of ``repeats``."""
    import torch

    from llmserver_amd.engine import Engine
    engine = Engine(model, None, max_new_tokens=1, max_batch_size=1, max_num_batched_tokens=max(cached, fresh),
                    kv_cache_num_blocks=2 * (-(-(cached + fresh) // page_size)) + 8, kv_cache_block_size=page_size, stream_text=False,
                    max_completed_requests=0, ignore_eos=True, enable_prefix_caching=True)
    generator = torch.Generator().manual_seed(seed)
    vocab = model.config.vocab_size
    earlier = torch.randint(0, vocab, (cached,), generator=generator).tolist()
    engine.add_request(None, prompt_token_ids=earlier)
    while engine.step():
        pass
    best = float("inf")
    for attempt in range(repeats + 1):
        request = engine.add_request(None, prompt_token_ids=earlier + torch.randint(0, vocab, (fresh,), generator=generator).tolist())
        torch.cuda.synchronize()
        start = time.perf_counter()
        more = engine.step()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - start
        assert not more and len(request.generated_token_ids) == 1, "the earlier turn's pages were not found in the cache"
        if attempt:
            best = min(best, elapsed)
    del engine
    torch.cuda.empty_cache()
    return best


def decode_point(model, page_size, batch, context, steps, warmup):
    """Tokens a second, milliseconds a step and GB/s of the bytes a step has to read (at the steps' mean context)."""
    seconds, _ = decode_through_engine(model, page_size, batch, context, steps, warmup)
    ms = 1000.0 * seconds / steps
    first, last = decode_step_bytes(model, batch, context - steps + 1), decode_step_bytes(model, batch, context)
    return batch * steps / seconds, ms, (first + last) / 2.0 / (ms * 1e-3) / 1e9


def main() -> int:
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--context", type=int, default=4096, help="context length the timed decode steps end at")
    parser.add_argument("--layers", type=int, default=0, help="fewer layers than the configuration has, if memory or time needs it (0: all)")
    parser.add_argument("--dtype", default="bfloat16", choices=("bfloat16", "float32"))
    parser.add_argument("--page-size", type=int, default=16)
    parser.add_argument("--prefill-tokens", type=int, default=2048)
    parser.add_argument("--no-points", action="store_true", help="skip the batch 1 / batch 64 points")
    parser.add_argument("--no-extra-points", action="store_true", help="skip the Qwen3-1.7B-sized mixed workload and the Qwen3-32B-sized batch")
    parser.add_argument("--no-prefill", action="store_true")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this single-GPU engine")
        return 2
    if args.context - args.steps - args.warmup < 1:
        parser.error("--context must exceed --steps + --warmup")

    import torch

    from llmserver_amd.engine.loading import parse_dtype

    dtype = parse_dtype(args.dtype)
    short = "bf16" if dtype == torch.bfloat16 else "fp32"
    model, config, full_layers = random_model(MODEL, args.layers, dtype)

    log(f"[bench] decode batch {args.batch}: {args.batch} prompts of {args.context - args.steps - args.warmup} tokens, then {args.warmup} + {args.steps} steps")
    value, ms_per_step, achieved = decode_point(model, args.page_size, args.batch, args.context, args.steps, args.warmup)
    result = {
        "metric": f"decode tok/s at batch {args.batch}, context {args.context} (Qwen3-8B-sized, random weights)", "value": round(value, 2),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": short, "data": "synthetic",
        "config": {"model": "qwen3-8b-sized", "layers": config.num_hidden_layers, "layers_full": full_layers,
                   "hidden": config.hidden_size, "heads": config.num_attention_heads, "kv_heads": config.num_key_value_heads,
                   "head_dim": config.head_dim, "intermediate": config.intermediate_size, "vocab": config.vocab_size,
                   "global_batch": args.batch, "seq_len": args.context, "prefill_tokens": args.prefill_tokens,
                   "page_size": args.page_size, "weights": "random N(0,0.02)", "timed_through": "Engine.step",
                   "parallelism": "single-gpu"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if not args.no_prefill:
        log(f"[bench] prefill of {args.prefill_tokens} tokens")
        seconds = prefill_through_engine(model, args.page_size, args.prefill_tokens)
        flops = prefill_flops(model, args.prefill_tokens)
        result["prefill"] = {"value": round(args.prefill_tokens / seconds, 1), "tokens": args.prefill_tokens,
                             "ms": round(1000.0 * seconds, 3),
                             "frac": round(flops / seconds / (MFMA_PEAK_TFLOPS[short] * 1e12), 4)}
    points = {}
    if not args.no_points:
        for batch, steps in ((1, min(args.steps, 64)), (64, min(args.steps, 32))):
            log(f"[bench] decode batch {batch}")
            rate, ms, gbs = decode_point(model, args.page_size, batch, args.context, steps, min(args.warmup, 4))
            points[f"decode_b{batch}"] = round(rate, 2)
            points[f"decode_b{batch}_ms_per_step"] = round(ms, 4)
            points[f"decode_b{batch}_hbm_frac"] = round(gbs / HBM_PEAK_GBS, 4)
        # further sizes of the same model: a short and a long prompt, and a few requests far into their contexts
        for tokens in (512, 8192):
            log(f"[bench] prefill of {tokens} tokens")
            seconds = prefill_through_engine(model, args.page_size, tokens)
            points[f"prefill_{tokens}_ms"] = round(1000.0 * seconds, 3)
            points[f"prefill_{tokens}_mfma_frac"] = round(prefill_flops(model, tokens) / seconds / (MFMA_PEAK_TFLOPS[short] * 1e12), 4)
        log("[bench] prefill of 16,384 tokens")
        seconds = prefill_through_engine(model, args.page_size, 16384, repeats=2)
        points["prefill_16384_ms"] = round(1000.0 * seconds, 3)
        points["prefill_16384_mfma_frac"] = round(prefill_flops(model, 16384) / seconds / (MFMA_PEAK_TFLOPS[short] * 1e12), 4)
        log("[bench] 128 new tokens behind 8,064 cached ones")
        points["turn_128_after_8064_ms"] = round(1000.0 * turn_through_engine(model, args.page_size, 8064, 128), 3)
        log("[bench] decode batch 4 at a context of 16,384")
        rate, ms, gbs = decode_point(model, args.page_size, 4, 16384, 32, 4)
        points["decode_b4_ctx16384"] = round(rate, 2)
        points["decode_b4_ctx16384_ms_per_step"] = round(ms, 4)
        points["decode_b4_ctx16384_hbm_frac"] = round(gbs / HBM_PEAK_GBS, 4)
        log("[bench] decode batch 8 at a context of 32,768")
        rate, ms, gbs = decode_point(model, args.page_size, 8, 32768, 32, 4)
        points["decode_b8_ctx32768"] = round(rate, 2)
        points["decode_b8_ctx32768_ms_per_step"] = round(ms, 4)
        points["decode_b8_ctx32768_hbm_frac"] = round(gbs / HBM_PEAK_GBS, 4)
        # The baseline's own decode workload: prompts of 2,048 tokens decoded greedily to 4,096 tokens in all, every
        # decoding step of the run timed (2,040 of them after 8 of warm-up; mean context 3,076).
        if args.context == 4096:
            for batch in (1, 8, 64):
                log(f"[bench] prompts of 2,048 tokens decoded to 4,096, batch {batch}")
                rate, ms, gbs = decode_point(model, args.page_size, batch, 4096, 2040, 8)
                points[f"decode_2048_to_4096_b{batch}"] = round(rate, 2)
                points[f"decode_2048_to_4096_b{batch}_hbm_frac"] = round(gbs / HBM_PEAK_GBS, 4)
    del model
    torch.cuda.empty_cache()
    if not args.no_points and not args.no_extra_points and dtype == torch.bfloat16 and not args.layers:
        points.update(extra_points(dtype, args.page_size))
    if points:
        result["points"] = points
    print(json.dumps(result), flush=True)
    return 0


def extra_points(dtype, page_size):
    """The two other workloads the baseline names, each on a random model of its own size."""
    import torch

    from llmserver_amd.cli.benchmark import mixed_workload
    from llmserver_amd.engine import Engine
    points = {}
    # 64 concurrent requests, prompts of 16 to 2,048 tokens, half of them behind one shared prefix of 512 tokens, 256 new
    # tokens each, continuous batching with chunked prefill (Qwen3-1.7B sizes).
    model, config, _ = random_model("qwen3-1.7b", 0, dtype)
    requests, high, new_tokens = 64, 2048, 256
    engine = Engine(model, None, max_new_tokens=new_tokens, max_batch_size=requests, max_num_batched_tokens=16384,
                    kv_cache_num_blocks=requests * (-(-(high + new_tokens) // page_size)) + 8, kv_cache_block_size=page_size,
                    stream_text=False, max_completed_requests=0, ignore_eos=True, enable_prefix_caching=True)
    engine.warmup_graphs(max_context=high + new_tokens)
    entry = mixed_workload(engine, config.vocab_size, requests, 16, high, 512, 0.5, new_tokens)
    log(f"[bench] mixed workload: {entry}")
    points["mixed_1p7b_64req_generated_tok_s"] = round(entry["generated_tok_s"], 1)
    points["mixed_1p7b_64req_total_s"] = round(entry["total_s"], 3)
    points["mixed_1p7b_64req_prefix_hit_tokens"] = int(entry["prefix_hit_tokens"])
    points["mixed_1p7b_64req_prompt_tokens"] = int(entry["prompt_tokens_total"])
    del engine
    # Short prompts on the same model, from a request's arrival to its first token: steps of this size are replayed from
    # graphs (launched one by one, the host would bound them).
    for tokens in (32, 128):
        points[f"first_token_1p7b_{tokens}_ms"] = round(1000.0 * prefill_through_engine(model, page_size, tokens, repeats=4), 3)
    del model
    torch.cuda.empty_cache()
    # Batch 16 behind prompts of 8,192 tokens (Qwen3-32B sizes): the decoding steps up to a context of 8,192 + 64.
    model, config, _ = random_model("qwen3-32b", 0, dtype)
    batch, context, steps, warmup = 16, 8192 + 64, 48, 4
    rate, ms, gbs = decode_point(model, page_size, batch, context, steps, warmup)
    points["decode_32b_b16_ctx8192"] = round(rate, 2)
    points["decode_32b_b16_ctx8192_ms_per_step"] = round(ms, 4)
    points["decode_32b_b16_ctx8192_hbm_frac"] = round(gbs / HBM_PEAK_GBS, 4)
    del model
    torch.cuda.empty_cache()
    return points


if __name__ == "__main__":
    sys.exit(main())
