"""Benchmark of the engine on token-id prompts, in the manner of the reference's
``benchmark_cuda.py`` (benchmark_cuda.py:1-13, 475-496): option names and
meanings follow it where it has them.

    python benchmark.py --model DIR --prompt-tokens 128,1024 --batch-sizes 1,8,32 --output-tokens 128
    python benchmark.py --random-config qwen3-8b --prompt-tokens 2048 --batch-sizes 1,8,64 --output-tokens 2048
    python benchmark.py --model DIR --prompt-token-ids 151644,872,198 --max-new-tokens 32 --repeats 3

With ``--prompt`` (text, if the model folder has a ``tokenizer.json``) or ``--prompt-token-ids`` it benchmarks one prompt
in the manner of the reference's ``benchmark.py`` (benchmark.py:68-88, 339-341): model load, time to
the first token, generation and decode throughput, medians over ``--repeats``.

For each (prompt length, batch size):
  * ttft_s  = time to generate 1 token for the whole batch (prefill latency)
  * total_s = time to generate ``--output-tokens`` tokens for the whole batch
  * decode tok/s = batch * (output_tokens - 1) / (total_s - ttft_s)
EOS is ignored, decoding is greedy unless ``--temperature`` is given, and every (prompt length,
batch size, repeat) gets its own seeded random token ids, so prefix caching cannot help
(benchmark_cuda.py:13, 32-38).  ``--random-config`` draws seeded random weights
on the device instead of reading a folder.
"""
from __future__ import annotations

import argparse
import json
import math
import statistics
import sys
import time

RANDOM_CONFIGS = {
    "tiny-a": dict(num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
                   intermediate_size=128, vocab_size=256, rope_theta=10000.0, rms_norm_eps=1e-6, tie_word_embeddings=True),
    "tiny-b": dict(num_hidden_layers=3, hidden_size=96, num_attention_heads=8, num_key_value_heads=2, head_dim=32,
                   intermediate_size=224, vocab_size=384, rope_theta=1e6, rms_norm_eps=1e-5, attention_bias=True),
    "qwen3-1.7b": dict(num_hidden_layers=28, hidden_size=2048, num_attention_heads=16, num_key_value_heads=8, head_dim=128,
                       intermediate_size=6144, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=True),
    "qwen3-8b": dict(num_hidden_layers=36, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
                     intermediate_size=12288, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6),
    "qwen3-14b": dict(num_hidden_layers=40, hidden_size=5120, num_attention_heads=40, num_key_value_heads=8, head_dim=128,
                      intermediate_size=17408, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6),
    "qwen3-32b": dict(num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, num_key_value_heads=8, head_dim=128,
                      intermediate_size=25600, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6),
}


def parse_ints(text):
    return [int(item) for item in text.split(",") if item.strip()]


def build_prompts(vocab, prompt_tokens, count, tag, seed):
    """Seeded uniform random token ids, different for every tag (they stand in for tokenised text)."""
    import hashlib

    import torch
    generator = torch.Generator().manual_seed(int.from_bytes(hashlib.sha256(f"{tag}:{seed}".encode()).digest()[:4], "little"))
    return [torch.randint(0, vocab, (prompt_tokens,), generator=generator).tolist() for _ in range(count)]


def run_once(engine, prompts, new_tokens):
    import torch
    engine.max_new_tokens = new_tokens
    torch.cuda.synchronize()
    start = time.perf_counter()
    requests = [engine.add_request(None, prompt_token_ids=prompt, max_new_tokens=new_tokens) for prompt in prompts]
    while engine.step():
        pass
    torch.cuda.synchronize()
    return time.perf_counter() - start, [list(r.generated_token_ids) for r in requests]


def mixed_workload(engine, vocab, requests, low, high, shared_prefix_tokens, shared_fraction, output_tokens, seed=0) -> dict:
    """``requests`` concurrent requests with prompt lengths uniform in [low, high], a fraction of them starting with
    one shared random prefix, ``output_tokens`` greedy tokens each, under continuous batching with chunked prefill.
    A short run first loads what a first run loads; the counters are the timed run's."""
    import random
    rng = random.Random(seed)
    prefix = build_prompts(vocab, shared_prefix_tokens, 1, "shared-prefix", seed)[0]
    prompts = []
    for index in range(requests):
        length = rng.randint(low, high)
        body = build_prompts(vocab, length, 1, f"mixed-{index}", seed)[0]
        if index < shared_fraction * requests and length > shared_prefix_tokens:
            body = prefix + body[shared_prefix_tokens:]
        prompts.append(body)
    rng.shuffle(prompts)
    run_once(engine, build_prompts(vocab, 64, min(4, engine.scheduler.max_batch_size), "warm-mixed", seed), 4)
    for key in ("steps", "decode_steps", "prefill_steps", "tokens", "prefix_hit_tokens", "preemptions"):
        engine.step_profile[key] = 0
    seconds, _ = run_once(engine, prompts, output_tokens)
    prompt_total = sum(len(p) for p in prompts)
    return {"workload": "mixed", "requests": requests, "prompt_tokens_total": prompt_total, "output_tokens": output_tokens,
            "total_s": seconds, "generated_tok_s": requests * output_tokens / seconds,
            "processed_tok_s": (prompt_total + requests * output_tokens) / seconds,
            "prefix_hit_tokens": engine.step_profile["prefix_hit_tokens"], "steps": engine.step_profile["steps"],
            "preemptions": engine.step_profile["preemptions"]}


def profile_engine(engine, vocab, prompt_lengths, batches, seed, out_path) -> None:
    """Kernel tables of a few decode steps (one row and the largest batch, replayed from graphs and launched one by
    one) and of prefills (the shortest prompts at the largest batch, the longest at up to eight), with the steps'
    wall-clock times beside them, written to ``out_path``: what the reference's ``--profile`` writes
    (benchmark_cuda.py:255-330 there)."""
    import torch
    from torch.profiler import ProfilerActivity, profile

    def kernel_table(run):
        with profile(activities=[ProfilerActivity.CPU, ProfilerActivity.CUDA]) as trace:
            run()
            torch.cuda.synchronize()
        return trace.key_averages().table(sort_by="cuda_time_total", row_limit=25, max_name_column_width=70)

    def steps(count):
        for _ in range(count):
            engine.step()
        torch.cuda.synchronize()

    lines = []
    graphs_possible = engine.runner.use_graphs
    for batch in sorted({1, max(batches)}):
        for graphs in ((False, True) if graphs_possible else (False,)):
            engine.runner.use_graphs = graphs
            engine.runner.drop_graphs()
            prompts = build_prompts(vocab, min(prompt_lengths), batch, f"profile-{batch}-{graphs}", seed)
            requests = [engine.add_request(None, prompt_token_ids=prompt, max_new_tokens=64) for prompt in prompts]
            steps(4)                                        # the prompts, then a few decoding steps (graphs are captured here)
            start = time.perf_counter()
            steps(5)
            step_ms = (time.perf_counter() - start) / 5 * 1000
            lines.append(f"===== decode batch={batch} graphs={graphs}: {step_ms:.3f} ms a step =====")
            lines.append(kernel_table(lambda: steps(5)))
            for request in requests:
                engine.cancel_request(request.request_id)
    engine.runner.use_graphs = graphs_possible
    engine.runner.drop_graphs()
    for prompt_length, batch in {(min(prompt_lengths), max(batches)), (max(prompt_lengths), min(8, max(batches)))}:
        def prefill(tag):
            prompts = build_prompts(vocab, prompt_length, batch, f"{tag}-{prompt_length}-{batch}", seed)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for prompt in prompts:
                engine.add_request(None, prompt_token_ids=prompt, max_new_tokens=1)
            t1 = time.perf_counter()
            count = 1
            while engine.step():
                count += 1
            torch.cuda.synchronize()
            return t1 - t0, time.perf_counter() - t1, count
        prefill("profile-warm")
        added, stepped, count = prefill("profile-timed")
        lines.append(f"===== prefill prompt={prompt_length} batch={batch}: add_request x{batch} {added * 1000:.1f} ms + {count} engine steps {stepped * 1000:.1f} ms =====")
        lines.append(kernel_table(lambda: prefill("profile-traced")))
    lines.append("===== step profile =====")
    lines.append(json.dumps(engine.step_profile))
    with open(out_path, "w") as handle:
        handle.write("\n".join(lines) + "\n")
    print(f"kernel tables written to {out_path}", flush=True)


def one_prompt(args, model, load_seconds) -> int:
    """One prompt, ``--repeats`` fresh requests: the reference's single-prompt statistics
    (benchmark.py:68-88)."""
    import os

    import torch

    from ..engine import Engine
    tokenizer = None
    if args.prompt is not None:
        path = os.path.join(args.model or "", "tokenizer.json")
        if not args.model or not os.path.isfile(path):
            print("--prompt needs a model folder with a tokenizer.json; pass --prompt-token-ids instead", file=sys.stderr)
            return 2
        from tokenizers import Tokenizer
        tokenizer = Tokenizer.from_file(path)
        prompt_ids = tokenizer.encode(args.prompt).ids
    else:
        prompt_ids = parse_ints(args.prompt_token_ids)
    if not prompt_ids or args.max_new_tokens <= 0:
        print("the prompt must hold at least one token and --max-new-tokens must be positive", file=sys.stderr)
        return 2
    blocks = math.ceil((len(prompt_ids) + args.max_new_tokens) / args.block_size) + 8
    engine = Engine(model, None, max_new_tokens=args.max_new_tokens, max_batch_size=1,
                    max_num_batched_tokens=max(args.max_num_batched_tokens, 1), prefill_chunk_size=args.prefill_chunk_size,
                    kv_cache_num_blocks=blocks, kv_cache_block_size=args.block_size, stream_text=False, max_completed_requests=0,
                    ignore_eos=False, temperature=args.temperature, seed=args.seed, enable_prefix_caching=False)
    run_once(engine, [prompt_ids], min(args.max_new_tokens, 4))               # graphs are captured before the clock starts
    results = []
    for _ in range(args.repeats):
        torch.cuda.synchronize()
        start = time.perf_counter()
        request = engine.add_request(None, prompt_token_ids=prompt_ids, max_new_tokens=args.max_new_tokens)
        first = None
        while engine.step():
            if first is None and request.generated_token_ids:
                first = time.perf_counter() - start
        torch.cuda.synchronize()
        seconds = time.perf_counter() - start
        results.append((list(request.generated_token_ids), seconds, first if first is not None else seconds))
    tokens, seconds, first = results[-1]
    print(f"\nPrompt: {args.prompt if args.prompt is not None else prompt_ids}")
    print(f"Response: {tokenizer.decode(tokens) if tokenizer is not None else tokens}")
    print(f"\nDevice: {torch.cuda.get_device_name(0)} | Model: {model.name}")
    print(f"Prompt tokens: {len(prompt_ids)} | Generated tokens: {len(tokens)}")
    print(f"Model load: {load_seconds:.2f} s | Generation: {seconds:.3f} s")
    print(f"Time to first token: {first:.4f} s")
    print(f"Generation throughput: {len(tokens) / seconds:.2f} tokens/s")
    if len(tokens) > 1:
        print(f"Decode throughput: {(len(tokens) - 1) / (seconds - first):.2f} tokens/s")
    if len(results) > 1:
        print(f"median over {len(results)} runs: Generation: {statistics.median(r[1] for r in results):.3f} s | "
              f"Time to first token: {statistics.median(r[2] for r in results):.4f} s")
        speeds = [(len(r[0]) - 1) / (r[1] - r[2]) for r in results if len(r[0]) > 1]
        if speeds:
            print(f"median decode throughput: {statistics.median(speeds):.2f} tokens/s")
    return 0


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--model", default=None, help="model folder (config.json + safetensors)")
    parser.add_argument("--random-config", default=None, choices=sorted(RANDOM_CONFIGS), help="seeded random weights of a named size instead of --model")
    parser.add_argument("--prompt", default=None, help="one prompt as text (needs tokenizer.json in the model folder)")
    parser.add_argument("--prompt-token-ids", default=None, help="one prompt as comma-separated token ids")
    parser.add_argument("--max-new-tokens", type=int, default=32, help="tokens to generate for --prompt / --prompt-token-ids")
    parser.add_argument("--prompt-tokens", default="128,1024")
    parser.add_argument("--batch-sizes", default="1,8,32")
    parser.add_argument("--output-tokens", type=int, default=128)
    parser.add_argument("--repeats", type=int, default=3)
    parser.add_argument("--dtype", default="bfloat16", choices=("bfloat16", "float32"))
    parser.add_argument("--custom-dtype", default=None, choices=("source", "fp32", "fp16"),
                        help="the reference's name of --dtype (benchmark.py:344): source = bfloat16 as stored, fp32 = float32; fp16 is not built")
    parser.add_argument("--device", default="cuda")
    parser.add_argument("--block-size", type=int, default=16)
    parser.add_argument("--max-num-batched-tokens", type=int, default=16384)
    parser.add_argument("--prefill-chunk-size", type=int, default=None)
    parser.add_argument("--temperature", type=float, default=0.0)
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument("--mixed-requests", type=int, default=0,
                        help="instead of the matrix: this many concurrent requests under continuous batching with chunked prefill")
    parser.add_argument("--mixed-prompt-range", default="16,2048", help="prompt lengths of the mixed workload, uniform in [lo, hi]")
    parser.add_argument("--shared-prefix-tokens", type=int, default=512, help="length of the prefix that some mixed requests share")
    parser.add_argument("--shared-fraction", type=float, default=0.5, help="fraction of mixed requests that start with the shared prefix")
    parser.add_argument("--max-batch-size", type=int, default=None, help="requests running at a time (default: the largest batch)")
    parser.add_argument("--profile", action="store_true",
                        help="print the engine's per-phase step counters and write kernel tables of decode steps and prefills to --profile-out")
    parser.add_argument("--profile-out", default="profile_kernels.txt", help="where --profile writes its kernel tables")
    parser.add_argument("--json", default=None, help="write the results to this file")
    args = parser.parse_args(argv)
    if (args.model is None) == (args.random_config is None):
        parser.error("pass exactly one of --model and --random-config")
    if args.custom_dtype == "fp16":
        parser.error("--custom-dtype fp16: this engine computes in bfloat16 (source) or float32 (fp32) only")
    if args.custom_dtype is not None:
        args.dtype = {"source": "bfloat16", "fp32": "float32"}[args.custom_dtype]

    import torch

    from ..config import config_from_dict
    from ..engine import Engine, load_model
    from ..engine.loading import parse_dtype
    from ..cache import CacheManager
    from ..weights import RandomInit, random_model_on_device

    started = time.perf_counter()
    if args.model:
        model = load_model(args.model, args.device, args.dtype)
    else:
        config = config_from_dict(dict(RANDOM_CONFIGS[args.random_config], model_type="qwen3"))
        model = random_model_on_device(config, args.device, parse_dtype(args.dtype), RandomInit(seed=args.seed, std=0.02))
        model.name = args.random_config
    torch.cuda.synchronize()
    print(f"loaded {model.name} in {time.perf_counter() - started:.1f} s", flush=True)
    vocab = model.config.vocab_size
    if args.prompt is not None or args.prompt_token_ids is not None:
        return one_prompt(args, model, time.perf_counter() - started)
    prompt_lengths, batches = parse_ints(args.prompt_tokens), parse_ints(args.batch_sizes)
    if args.mixed_requests:
        low, high = parse_ints(args.mixed_prompt_range)
        prompt_lengths, batches = [high], [args.max_batch_size or args.mixed_requests]
    max_batch, max_length = max(batches), max(prompt_lengths) + args.output_tokens
    bytes_per_block = CacheManager.bytes_per_token(model.cache_specs(), model.dtype) * args.block_size
    wanted = max_batch * math.ceil(max_length / args.block_size) + 8          # benchmark_cuda.py:107-111
    wanted = min(wanted, int(torch.cuda.mem_get_info()[0] * 0.8 // max(1, bytes_per_block)))
    engine = Engine(model, None, max_new_tokens=1, max_batch_size=max_batch,
                    max_num_batched_tokens=max(args.max_num_batched_tokens, max_batch), prefill_chunk_size=args.prefill_chunk_size,
                    kv_cache_num_blocks=wanted, kv_cache_block_size=args.block_size, stream_text=False, max_completed_requests=0,
                    ignore_eos=True, temperature=args.temperature, seed=args.seed, enable_prefix_caching=True)
    results = []
    if args.mixed_requests:
        # A server captures its decode graphs at start-up, before requests come (server.py:332 in the reference):
        # so does this workload, which stands for one.
        engine.warmup_graphs(max_context=high + args.output_tokens)
        entry = mixed_workload(engine, vocab, args.mixed_requests, low, high, args.shared_prefix_tokens, args.shared_fraction,
                               args.output_tokens, args.seed)
        print(f"mixed: {args.mixed_requests} requests, {entry['prompt_tokens_total']} prompt tokens ({entry['prefix_hit_tokens']} served from cached prefix pages), "
              f"{args.output_tokens} new tokens each: {entry['total_s']:.3f} s, {entry['generated_tok_s']:.1f} generated tok/s, "
              f"{entry['processed_tok_s']:.1f} processed tok/s, {entry['steps']} steps, {entry['preemptions']} preemptions", flush=True)
        results.append(entry)
        prompt_lengths = []
    for prompt_length in prompt_lengths:
        for batch in batches:
            entry = {"prompt_tokens": prompt_length, "batch": batch, "output_tokens": args.output_tokens}
            try:
                if batch * (prompt_length + args.output_tokens) > wanted * args.block_size:
                    raise MemoryError("KV cache too small for this configuration")
                # One whole run first, as the reference warms up (benchmark_cuda.py:208 there): every graph the timed
                # runs replay is captured before the clock starts.
                run_once(engine, build_prompts(vocab, prompt_length, batch, f"warm-{prompt_length}-{batch}", args.seed), args.output_tokens)
                ttft, total, tokens = [], [], None
                for repeat in range(args.repeats):
                    seconds, _ = run_once(engine, build_prompts(vocab, prompt_length, batch, f"t1-{prompt_length}-{batch}-{repeat}", args.seed), 1)
                    ttft.append(seconds)
                for repeat in range(args.repeats):
                    seconds, generated = run_once(engine, build_prompts(vocab, prompt_length, batch, f"tn-{prompt_length}-{batch}-{repeat}", args.seed), args.output_tokens)
                    total.append(seconds)
                    tokens = tokens or generated
                ttft_s, total_s = statistics.median(ttft), statistics.median(total)
                decode_s = max(total_s - ttft_s, 1e-9)
                entry.update(ttft_s=ttft_s, total_s=total_s, decode_tok_s=batch * (args.output_tokens - 1) / decode_s,
                             e2e_tok_s=batch * args.output_tokens / total_s, prefill_tok_s=batch * prompt_length / ttft_s,
                             ms_per_token=1000 * decode_s / max(args.output_tokens - 1, 1), tokens=tokens,
                             peak_alloc_gb=round(torch.cuda.max_memory_allocated() / 2 ** 30, 2))
                print(f"prompt {prompt_length:6d}  batch {batch:3d}:  ttft {ttft_s * 1000:9.2f} ms   decode {entry['decode_tok_s']:10.1f} tok/s   "
                      f"prefill {entry['prefill_tok_s']:10.1f} tok/s   end-to-end {entry['e2e_tok_s']:10.1f} tok/s", flush=True)
            except Exception as error:            # record per-configuration failures (e.g. out of memory) and go on
                entry["error"] = f"{type(error).__name__}: {error}"
                print(f"prompt {prompt_length:6d}  batch {batch:3d}:  {entry['error']}", flush=True)
            results.append(entry)
    if args.profile:
        print("step profile:", json.dumps(engine.step_profile), flush=True)
        engine.max_new_tokens = 64
        profile_engine(engine, vocab, prompt_lengths or [high], batches, args.seed, args.profile_out)
    report = {"model": model.name, "dtype": args.dtype, "block_size": args.block_size, "kv_blocks": wanted, "gpu": torch.cuda.get_device_name(0),
              "torch": torch.__version__, "results": results, "step_profile": engine.step_profile}
    if args.json:
        with open(args.json, "w") as handle:
            json.dump(report, handle)
    return 0


if __name__ == "__main__":
    sys.exit(main())
