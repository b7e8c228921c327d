"""The benchmark command line on the GPU: the matrix over prompt lengths and batch sizes, one prompt with the
reference's statistics, the mixed workload; tokens of a greedy run against the plain implementation."""
import json

import pytest

import plain_qwen3 as plain
from helpers import model_folder, plain_model, random_tokens
from tiny_configs import CASES

pytestmark = pytest.mark.gpu


def test_matrix_one_prompt_and_mixed_workload(tmp_path, capsys):
    from llmserver_amd.cli import benchmark
    case = "A"
    raw, _, page = CASES[case]
    folder = model_folder(case)
    report = tmp_path / "report.json"
    assert benchmark.main(["--model", folder, "--dtype", "float32", "--prompt-tokens", "9,40", "--batch-sizes", "1,3", "--output-tokens", "6",
                           "--repeats", "1", "--block-size", str(page), "--json", str(report)]) == 0
    results = json.loads(report.read_text())["results"]
    assert [(r["prompt_tokens"], r["batch"]) for r in results] == [(9, 1), (9, 3), (40, 1), (40, 3)]
    assert all(r["decode_tok_s"] > 0 and r["ttft_s"] > 0 and len(r["tokens"]) == r["batch"] and len(r["tokens"][0]) == 6 for r in results)
    # the matrix's prompts are seeded: the same ids here, through the plain implementation
    config, tensors = plain_model(case)
    prompt = benchmark.matrix_prompts(raw["vocab_size"], 9, 1, "whole-run", 0, 0)[0]
    assert results[0]["tokens"][0] == plain.greedy_generate(config, tensors, prompt, 6)
    capsys.readouterr()
    prompt = random_tokens(raw["vocab_size"], 7, 3)
    assert benchmark.main(["--model", folder, "--custom-dtype", "fp32", "--prompt-token-ids", ",".join(map(str, prompt)), "--max-new-tokens", "5",
                           "--repeats", "2", "--block-size", str(page)]) == 0
    printed = capsys.readouterr().out
    assert f"response: {plain.greedy_generate(config, tensors, prompt, 5)}" in printed
    assert "7 in the prompt, 5 generated" in printed and "first token:" in printed and "medians of 2 runs: first token" in printed
    assert benchmark.main(["--model", folder, "--prompt", "text without a tokenizer"]) == 2
    assert benchmark.main(["--random-config", "tiny-b", "--mixed-requests", "6", "--mixed-prompt-range", "4,40", "--shared-prefix-tokens", "16",
                           "--output-tokens", "5", "--block-size", "8", "--max-num-batched-tokens", "64", "--profile",
                           "--profile-out", str(tmp_path / "kernels.txt")]) == 0
    printed = capsys.readouterr().out
    assert "mixed: 6 requests" in printed and "step profile:" in printed and "decode_by_rows" in printed
    tables = (tmp_path / "kernels.txt").read_text()
    assert "decode batch=1 graphs=True" in tables and "decode batch=6 graphs=False" in tables and "prefill prompt=40" in tables
    assert "paged_attention" in tables and "gemm_skinny" in tables           # this repository's kernels, by name, with their times


def test_bench_prints_one_line_with_every_part_and_refuses_more_gpus():
    """``bench.py`` as the driver runs it, on two layers of the benchmark's sizes so that it takes seconds: one JSON line
    whose parts are all there (value, roofline, prefill, points at further sizes); more than one GPU: one line, exit 2."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    print("bench.py on two layers", flush=True)
    done = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--layers", "2", "--steps", "4", "--warmup", "1", "--context", "256"],
                          capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-3000:]
    lines = [line for line in done.stdout.splitlines() if line.strip()]
    assert len(lines) == 1
    record = json.loads(lines[0])
    assert record["n_gpus"] == 1 and record["steps"] == 4 and record["warmup"] == 1 and record["value"] > 0 and record["unit"] == "tokens/s"
    assert record["config"]["layers"] == 2 and record["config"]["layers_full"] == 36 and len(record["config"]) <= 20
    assert all(not isinstance(value, (dict, list)) for value in record["config"].values())
    assert record["roofline"]["bound"] == "hbm" and 0 < record["roofline"]["frac"] < 1
    assert record["prefill"]["tokens"] == 2048 and record["prefill"]["ms"] > 0 and 0 < record["prefill"]["frac"] < 1
    for key in ("decode_b1", "decode_b64", "decode_b64_ms_per_step", "prefill_512_ms", "prefill_8192_ms", "decode_b4_ctx16384"):
        assert record["points"][key] > 0, key
    assert not any(key.startswith("mixed_") for key in record["points"])       # fewer layers: the other models' points are left out
    more = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert more.returncode == 2 and len(more.stdout.strip().splitlines()) == 1
