"""Decode and prefill throughput of the engine on one MI355X, with random weights.

    python bench.py --gpus 1 --steps K --warmup W

Default workload: the Qwen3-8B-sized configuration (36 layers, hidden 4096, 32 query heads, 8 KV
heads, head size 128, intermediate 12288, vocabulary 151936, untied head), bfloat16, a batch of 8
requests decoding at a context of 4,096 tokens.  A "step" is one decode step of the whole batch:
build the batch, run the model against the paged cache, sample greedily, return the token ids.
Prints ONE JSON line: ``value`` is decoded tokens per second; ``prefill`` times one 2,048-token
prompt; ``roofline`` relates the bytes a decode step has to read (every weight once, plus the
cache of the live requests) to the published HBM bandwidth; ``points`` holds batch 1 and 64.
Token ids are seeded uniform random numbers (synthetic data), weights seeded normal.
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
QWEN3_8B = dict(model_type="qwen3", num_hidden_layers=36, hidden_size=4096, num_attention_heads=32,
                num_key_value_heads=8, head_dim=128, intermediate_size=12288, vocab_size=151936, rope_theta=1e6,
                rms_norm_eps=1e-6, attention_bias=False, tie_word_embeddings=False, max_position_embeddings=40960)
FULL_LAYERS = QWEN3_8B["num_hidden_layers"]


def log(*args):
    print(*args, file=sys.stderr, flush=True)


def weight_bytes(config, elem):
    c = config
    per_layer = c.hidden_size * (c.num_attention_heads + 2 * c.num_key_value_heads) * c.head_dim \
        + c.num_attention_heads * c.head_dim * c.hidden_size + 3 * c.hidden_size * c.intermediate_size
    return elem * (c.num_hidden_layers * per_layer + c.vocab_size * c.hidden_size)


def kv_bytes_per_token(config, elem):
    return 2 * config.num_key_value_heads * config.head_dim * elem * config.num_hidden_layers


def prefill_flops(config, tokens):
    c = config
    per_layer = c.hidden_size * (c.num_attention_heads + 2 * c.num_key_value_heads) * c.head_dim \
        + c.num_attention_heads * c.head_dim * c.hidden_size + 3 * c.hidden_size * c.intermediate_size
    gemm = 2.0 * tokens * per_layer * c.num_hidden_layers + 2.0 * c.vocab_size * c.hidden_size
    attention = 2.0 * c.num_attention_heads * c.head_dim * tokens * (tokens + 1) * c.num_hidden_layers
    return gemm + attention


class DecodeBench:
    """Holds B requests at a given context in the engine's cache and steps them."""

    def __init__(self, model, page_size, batch, context, final_context, prompt_chunk=2048, seed=0):
        import torch

        from llmserver_amd.cache import CacheManager
        from llmserver_amd.engine import ModelRunner, StepEntry
        from llmserver_amd.sampling import Sampler

        self.torch, self.StepEntry = torch, StepEntry
        self.batch = batch
        pages = batch * (-(-(final_context + 8) // page_size)) + 8
        self.cache = CacheManager(model.cache_specs(), page_size, pages, device=model.device, dtype=model.dtype)
        self.runner = ModelRunner(model, self.cache)
        self.sampler = Sampler(self.runner.ops, model.device)
        generator = torch.Generator().manual_seed(seed)
        self.ids = [f"r{i}" for i in range(batch)]
        self.last = []
        vocab = model.config.vocab_size
        for rid in self.ids:
            self.cache.open(rid)
        # Fill every request's cache up to `context` tokens with real prefill steps.
        for rid in self.ids:
            done = 0
            while done < context:
                n = min(prompt_chunk, context - done)
                tokens = torch.randint(0, vocab, (n,), generator=generator).tolist()
                self.runner.step([StepEntry(rid, tokens, [])])
                done += n
        self.last = torch.randint(0, vocab, (batch,), generator=generator).tolist()
        torch.cuda.synchronize()

    def step(self, more_follow=True):
        entries = [self.StepEntry(rid, [token], [0]) for rid, token in zip(self.ids, self.last)]
        logits = self.runner.step(entries)
        sampled = self.sampler.launch(logits, [0.0] * self.batch, [0.0] * self.batch)
        # As the engine does while it knows that all requests go on: the next step is laid out on the host while the
        # GPU runs this one, and started with the sampled tokens still on the device.
        if more_follow and self.runner.prepare_ahead(self.ids):
            self.runner.launch_ahead(sampled.device)
        self.last = sampled.tolist()

    def run(self, steps, warmup):
        """Seconds for exactly ``steps`` decode steps: the last warm-up step starts nothing that the timed steps would
        find done, and the last timed step starts nothing that would run beyond them."""
        torch = self.torch
        for index in range(warmup):
            self.step(more_follow=index + 1 < warmup)
        torch.cuda.synchronize()
        start = time.perf_counter()
        for index in range(steps):
            self.step(more_follow=index + 1 < steps)
        torch.cuda.synchronize()
        return time.perf_counter() - start

    def close(self):
        for rid in self.ids:
            self.cache.close(rid)
        del self.runner, self.cache
        self.torch.cuda.empty_cache()


def time_prefill(model, page_size, tokens, repeats=3, seed=1):
    import torch

    from llmserver_amd.cache import CacheManager
    from llmserver_amd.engine import ModelRunner, StepEntry

    cache = CacheManager(model.cache_specs(), page_size, -(-tokens // page_size) + 4, device=model.device, dtype=model.dtype)
    runner = ModelRunner(model, cache)
    generator = torch.Generator().manual_seed(seed)
    best = float("inf")
    for attempt in range(repeats + 1):
        prompt = torch.randint(0, model.config.vocab_size, (tokens,), generator=generator).tolist()
        cache.open("p")
        torch.cuda.synchronize()
        start = time.perf_counter()
        logits = runner.step([StepEntry("p", prompt, [tokens - 1])])
        int(torch.argmax(logits[0]))
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - start
        cache.close("p")
        if attempt:
            best = min(best, elapsed)
    return best


def main() -> int:
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--context", type=int, default=4096, help="context length the timed decode steps end at")
    parser.add_argument("--layers", type=int, default=FULL_LAYERS, help="fewer layers than the configuration has, if memory or time needs it")
    parser.add_argument("--dtype", default="bfloat16", choices=("bfloat16", "float32"))
    parser.add_argument("--page-size", type=int, default=16)
    parser.add_argument("--prefill-tokens", type=int, default=2048)
    parser.add_argument("--no-points", action="store_true", help="skip the batch 1 / batch 64 points")
    parser.add_argument("--no-prefill", action="store_true")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this single-GPU engine")
        return 2

    import torch

    from llmserver_amd.config import config_from_dict
    from llmserver_amd.engine.loading import parse_dtype
    from llmserver_amd.kernels import default_ops
    from llmserver_amd.weights import RandomInit, random_model_on_device

    raw = dict(QWEN3_8B, num_hidden_layers=args.layers)
    config = config_from_dict(raw)
    dtype = parse_dtype(args.dtype)
    short = "bf16" if dtype == torch.bfloat16 else "fp32"
    elem = 2 if dtype == torch.bfloat16 else 4
    default_ops().preload([config.head_dim], dtype)
    log(f"[bench] drawing random weights: {weight_bytes(config, elem) / 1e9:.2f} GB")
    model = random_model_on_device(config, "cuda:0", dtype, RandomInit(seed=0, std=0.02))
    model.name = "qwen3-8b-random"

    start_context = args.context - args.steps - args.warmup
    if start_context < 1:
        parser.error("--context must exceed --steps + --warmup")

    def decode_rate(batch, steps, warmup):
        log(f"[bench] decode batch {batch}: filling {batch} x {args.context - steps - warmup} tokens of cache")
        bench = DecodeBench(model, args.page_size, batch, args.context - steps - warmup, args.context)
        log(f"[bench] decode batch {batch}: timing {steps} steps")
        elapsed = bench.run(steps, warmup)
        bench.close()
        return elapsed

    elapsed = decode_rate(args.batch, args.steps, args.warmup)
    ms_per_step = 1000.0 * elapsed / args.steps
    value = args.batch * args.steps / elapsed
    mean_context = args.context - args.steps / 2.0
    step_bytes = weight_bytes(config, elem) + args.batch * mean_context * kv_bytes_per_token(config, elem)
    achieved = step_bytes / (ms_per_step * 1e-3) / 1e9
    result = {
        "metric": f"decode tok/s at batch {args.batch}, context {args.context} (Qwen3-8B-sized, random weights)", "value": round(value, 2),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": short, "data": "synthetic",
        "config": {"model": "qwen3-8b-sized", "layers": config.num_hidden_layers, "layers_full": FULL_LAYERS,
                   "hidden": config.hidden_size, "heads": config.num_attention_heads, "kv_heads": config.num_key_value_heads,
                   "head_dim": config.head_dim, "intermediate": config.intermediate_size, "vocab": config.vocab_size,
                   "global_batch": args.batch, "seq_len": args.context, "prefill_tokens": args.prefill_tokens,
                   "page_size": args.page_size, "weights": "random N(0,0.02)", "parallelism": "single-gpu"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if not args.no_prefill:
        log(f"[bench] prefill of {args.prefill_tokens} tokens")
        seconds = time_prefill(model, args.page_size, args.prefill_tokens)
        flops = prefill_flops(config, args.prefill_tokens)
        result["prefill"] = {"value": round(args.prefill_tokens / seconds, 1), "tokens": args.prefill_tokens,
                             "ms": round(1000.0 * seconds, 3),
                             "frac": round(flops / seconds / (MFMA_PEAK_TFLOPS[short] * 1e12), 4)}
    if not args.no_points:
        points = {}
        for batch, steps in ((1, min(args.steps, 64)), (64, min(args.steps, 32))):
            seconds = decode_rate(batch, steps, min(args.warmup, 4))
            points[f"decode_b{batch}"] = round(batch * steps / seconds, 2)
        result["points"] = points
    print(json.dumps(result), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
