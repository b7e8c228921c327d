"""Benchmark of the engine on token-id prompts, in the manner of the reference's
``benchmark_cuda.py`` (benchmark_cuda.py:1-13, 475-496): option names and
meanings follow it where it has them.

    python benchmark.py --model DIR --prompt-tokens 128,1024 --batch-sizes 1,8,32 --output-tokens 128
    python benchmark.py --random-config qwen3-8b --prompt-tokens 2048 --batch-sizes 1,8,64 --output-tokens 2048
    python benchmark.py --model DIR --prompt-token-ids 151644,872,198 --max-new-tokens 32 --repeats 3

With ``--prompt`` (text, if the model folder has a ``tokenizer.json``) or ``--prompt-token-ids`` it benchmarks one prompt
in the manner of the reference's ``benchmark.py`` (benchmark.py:68-88, 339-341): model load, time to
the first token, generation and decode throughput, medians over ``--repeats``.

The matrix times two things per (prompt length, batch size), each the median of ``--repeats`` runs on fresh prompts
(the definitions are the reference's, benchmark_cuda.py:8-13): ``ttft_s``, a run that generates one
token per request, i.e. the prompts' way to their first tokens; and ``total_s``, a run that generates ``--output-tokens``.
What lies between them is decoding: ``decode_tok_s = batch * (output_tokens - 1) / (total_s - ttft_s)``.  EOS is
ignored, decoding is greedy unless ``--temperature`` is given, and every run's prompts are seeded random token ids of
their own, so that cached prefix pages cannot help.  ``--random-config`` draws seeded random weights on the device
instead of reading a folder.
"""
from __future__ import annotations

import argparse
import dataclasses
import json
import statistics
import sys
import time
from typing import List, Optional

from ..config.named_sizes import NAMED_SIZES


def int_list(text: str) -> List[int]:
    """An option's value ``"128, 1024"`` as ``[128, 1024]`` (an ``argparse`` type: a bad item is the option's error)."""
    try:
        return [int(item) for item in text.replace(" ", "").split(",") if item]
    except ValueError:
        raise argparse.ArgumentTypeError(f"expected integers separated by commas, got {text!r}") from None


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


@dataclasses.dataclass
class PromptRun:
    """One request from its arrival to its last token."""
    tokens: List[int]
    seconds: float
    first_token_seconds: float

    @property
    def decode_rate(self) -> Optional[float]:
        """Tokens a second after the first one; None for a run of one token."""
        rest = len(self.tokens) - 1
        return rest / max(self.seconds - self.first_token_seconds, 1e-9) if rest > 0 else None


def time_one_prompt(engine, prompt_ids, new_tokens) -> PromptRun:
    import torch
    torch.cuda.synchronize()
    arrived = time.perf_counter()
    request = engine.add_request(None, prompt_token_ids=prompt_ids, max_new_tokens=new_tokens)
    first = None
    while engine.step():
        if first is None and request.generated_token_ids:
            first = time.perf_counter()
    torch.cuda.synchronize()
    finished = time.perf_counter()
    return PromptRun(list(request.generated_token_ids), finished - arrived, (first or finished) - arrived)


def one_prompt(args, model, load_seconds) -> int:
    """One prompt, ``--repeats`` fresh requests, and what the reference's single-prompt benchmark reports of them
    (benchmark.py:68-88): load time, time to the first token, the whole generation, throughput overall
    and of decoding alone, medians when there are several runs."""
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
        prompt_ids = args.prompt_token_ids
    if not prompt_ids or args.max_new_tokens <= 0:
        print("the prompt must hold at least one token and --max-new-tokens must be positive", file=sys.stderr)
        return 2
    engine = Engine(model, None, max_new_tokens=args.max_new_tokens, max_batch_size=1,
                    max_num_batched_tokens=max(args.max_num_batched_tokens, 1), prefill_chunk_size=args.prefill_chunk_size,
                    kv_cache_num_blocks=pool_pages(model, args.block_size, 1, len(prompt_ids) + args.max_new_tokens),
                    kv_cache_block_size=args.block_size, stream_text=False, max_completed_requests=0,
                    ignore_eos=False, temperature=args.temperature, seed=args.seed, enable_prefix_caching=False)
    run_once(engine, [prompt_ids], min(args.max_new_tokens, 4))               # graphs are captured before the clock starts
    runs = [time_one_prompt(engine, prompt_ids, args.max_new_tokens) for _ in range(args.repeats)]
    last = runs[-1]
    shown = {"prompt": args.prompt if args.prompt is not None else prompt_ids,
             "response": tokenizer.decode(last.tokens) if tokenizer is not None else last.tokens,
             "model": f"{model.name} ({args.dtype}) on {torch.cuda.get_device_name(0)}",
             "tokens": f"{len(prompt_ids)} in the prompt, {len(last.tokens)} generated",
             "load": f"{load_seconds:.2f} s",
             "first token": f"{last.first_token_seconds * 1000:.2f} ms after the request arrived",
             "whole run": f"{last.seconds:.3f} s, {len(last.tokens) / last.seconds:.2f} tokens/s"}
    if last.decode_rate is not None:
        shown["decoding"] = f"{last.decode_rate:.2f} tokens/s after the first token"
    if len(runs) > 1:
        medians = [f"first token {statistics.median(run.first_token_seconds for run in runs) * 1000:.2f} ms",
                   f"whole run {statistics.median(run.seconds for run in runs):.3f} s"]
        rates = [run.decode_rate for run in runs if run.decode_rate is not None]
        if rates:
            medians.append(f"decoding {statistics.median(rates):.2f} tokens/s")
        shown[f"medians of {len(runs)} runs"] = ", ".join(medians)
    print()
    for label, value in shown.items():
        print(f"{label:>18}: {value}")
    return 0


def pool_pages(model, block_size: int, batch: int, tokens_per_request: int, memory_share: float = 0.85) -> int:
    """Pages for ``batch`` requests that each grow to ``tokens_per_request`` tokens: their own pages, and the spare page
    per running request that the scheduler keeps free before it admits another; never more than ``memory_share`` of the
    device memory that is free now (activations and graphs need the rest)."""
    import torch

    from ..cache import CacheManager
    per_request = -(-tokens_per_request // block_size) + 1
    page_bytes = max(1, CacheManager.bytes_per_token(model.cache_specs(), model.dtype) * block_size)
    fitting = int(memory_share * torch.cuda.mem_get_info()[0]) // page_bytes
    return max(1, min(batch * per_request, fitting))


@dataclasses.dataclass
class Measurement:
    """One cell of the matrix: runs to the first token and runs to ``output_tokens`` tokens, on fresh prompts each."""
    prompt_tokens: int
    batch: int
    output_tokens: int
    first_token_runs: List[float] = dataclasses.field(default_factory=list)     # seconds of runs that generate one token per request
    whole_runs: List[float] = dataclasses.field(default_factory=list)           # seconds of runs that generate output_tokens
    tokens: Optional[List[List[int]]] = None                                    # what the first whole run generated
    peak_memory_bytes: int = 0
    failure: Optional[str] = None

    @property
    def ttft_s(self) -> float:
        return statistics.median(self.first_token_runs)

    @property
    def total_s(self) -> float:
        return statistics.median(self.whole_runs)

    @property
    def decode_s(self) -> float:
        """What a whole run takes beyond the first tokens."""
        return max(self.total_s - self.ttft_s, 1e-9)

    @property
    def decode_tok_s(self) -> float:
        return self.batch * (self.output_tokens - 1) / self.decode_s

    @property
    def prefill_tok_s(self) -> float:
        return self.batch * self.prompt_tokens / self.ttft_s

    @property
    def end_to_end_tok_s(self) -> float:
        return self.batch * self.output_tokens / self.total_s

    def record(self) -> dict:
        """The cell as it goes into the ``--json`` report."""
        cell = {"prompt_tokens": self.prompt_tokens, "batch": self.batch, "output_tokens": self.output_tokens}
        if self.failure is not None:
            return dict(cell, error=self.failure)
        return dict(cell, ttft_s=self.ttft_s, total_s=self.total_s, decode_tok_s=self.decode_tok_s, prefill_tok_s=self.prefill_tok_s,
                    end_to_end_tok_s=self.end_to_end_tok_s, decode_ms_per_token=1000 * self.decode_s / max(self.output_tokens - 1, 1),
                    tokens=self.tokens, peak_memory_gib=round(self.peak_memory_bytes / 2 ** 30, 2))

    def line(self) -> str:
        where = f"{self.batch:3d} x {self.prompt_tokens:6d} tokens"
        if self.failure is not None:
            return f"{where}: {self.failure}"
        return (f"{where}: first tokens after {self.ttft_s * 1000:9.2f} ms ({self.prefill_tok_s:10.1f} tok/s), "
                f"decoding {self.decode_tok_s:10.1f} tok/s, end to end {self.end_to_end_tok_s:10.1f} tok/s")


def matrix_prompts(vocab, prompt_tokens, batch, phase, repeat, seed):
    """The prompts of one run of one cell; ``phase``: "warm-up", "first-token" or "whole-run"."""
    return build_prompts(vocab, prompt_tokens, batch, f"{phase}/{prompt_tokens}x{batch}/{repeat}", seed)


def measure(engine, vocab, prompt_tokens, batch, output_tokens, repeats, seed, pool_tokens) -> Measurement:
    """Fill one cell.  A cell that cannot run (the pool is too small for it, memory runs out) says so in ``failure``
    and the matrix goes on."""
    import torch
    cell = Measurement(prompt_tokens, batch, output_tokens)
    needed = batch * (prompt_tokens + output_tokens)
    if needed > pool_tokens:
        cell.failure = f"needs {needed} tokens of cache, the pool holds {pool_tokens}"
        return cell
    try:
        # A whole run first, untimed: every graph that the timed runs replay is captured then
        # (the reference warms up the same way, benchmark_cuda.py:208).
        run_once(engine, matrix_prompts(vocab, prompt_tokens, batch, "warm-up", 0, seed), output_tokens)
        for repeat in range(repeats):
            cell.first_token_runs.append(run_once(engine, matrix_prompts(vocab, prompt_tokens, batch, "first-token", repeat, seed), 1)[0])
        for repeat in range(repeats):
            seconds, generated = run_once(engine, matrix_prompts(vocab, prompt_tokens, batch, "whole-run", repeat, seed), output_tokens)
            cell.whole_runs.append(seconds)
            cell.tokens = cell.tokens or generated
        cell.peak_memory_bytes = torch.cuda.max_memory_allocated()
    except (RuntimeError, MemoryError, BufferError) as error:
        cell.failure = f"{type(error).__name__}: {error}"
    return cell


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--model", default=None, help="model folder (config.json + safetensors)")
    parser.add_argument("--random-config", default=None, choices=sorted(NAMED_SIZES), help="seeded random weights of a named size instead of --model")
    parser.add_argument("--prompt", default=None, help="one prompt as text (needs tokenizer.json in the model folder)")
    parser.add_argument("--prompt-token-ids", default=None, type=int_list, help="one prompt as comma-separated token ids")
    parser.add_argument("--max-new-tokens", type=int, default=32, help="tokens to generate for --prompt / --prompt-token-ids")
    parser.add_argument("--prompt-tokens", default=[128, 1024], type=int_list)
    parser.add_argument("--batch-sizes", default=[1, 8, 32], type=int_list)
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
    parser.add_argument("--mixed-prompt-range", default=[16, 2048], type=int_list, help="prompt lengths of the mixed workload, uniform in [lo, hi]")
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
    if len(args.mixed_prompt_range) != 2:
        parser.error("--mixed-prompt-range takes two numbers: lo,hi")

    import torch

    from ..config import named_config
    from ..engine import Engine, load_model
    from ..engine.loading import parse_dtype
    from ..weights import RandomInit, random_model_on_device

    started = time.perf_counter()
    if args.model:
        model = load_model(args.model, args.device, args.dtype)
    else:
        model = random_model_on_device(named_config(args.random_config), args.device, parse_dtype(args.dtype), RandomInit(seed=args.seed, std=0.02))
        model.name = args.random_config
    torch.cuda.synchronize()
    print(f"loaded {model.name} in {time.perf_counter() - started:.1f} s", flush=True)
    vocab = model.config.vocab_size
    if args.prompt is not None or args.prompt_token_ids is not None:
        return one_prompt(args, model, time.perf_counter() - started)
    prompt_lengths, batches = args.prompt_tokens, args.batch_sizes
    if args.mixed_requests:
        low, high = args.mixed_prompt_range
        prompt_lengths, batches = [high], [args.max_batch_size or args.mixed_requests]
    pages = pool_pages(model, args.block_size, max(batches), max(prompt_lengths) + args.output_tokens)
    engine = Engine(model, None, max_new_tokens=1, max_batch_size=max(batches),
                    max_num_batched_tokens=max(args.max_num_batched_tokens, max(batches)), prefill_chunk_size=args.prefill_chunk_size,
                    kv_cache_num_blocks=pages, kv_cache_block_size=args.block_size, stream_text=False, max_completed_requests=0,
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
            cell = measure(engine, vocab, prompt_length, batch, args.output_tokens, args.repeats, args.seed, pages * args.block_size)
            print(cell.line(), flush=True)
            results.append(cell.record())
    if args.profile:
        print("step profile:", json.dumps(engine.step_profile), flush=True)
        engine.max_new_tokens = 64
        profile_engine(engine, vocab, prompt_lengths or [high], batches, args.seed, args.profile_out)
    report = {"model": model.name, "dtype": args.dtype, "block_size": args.block_size, "kv_blocks": pages, "gpu": torch.cuda.get_device_name(0),
              "torch": torch.__version__, "results": results, "step_profile": engine.step_profile}
    if args.json:
        with open(args.json, "w") as handle:
            json.dump(report, handle)
    return 0


if __name__ == "__main__":
    sys.exit(main())
