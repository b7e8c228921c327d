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
    prompt = benchmark.build_prompts(raw["vocab_size"], 9, 1, "tn-9-1-0", 0)[0]
    assert results[0]["tokens"][0] == plain.greedy_generate(config, tensors, prompt, 6)
    capsys.readouterr()
    prompt = random_tokens(raw["vocab_size"], 7, 3)
    assert benchmark.main(["--model", folder, "--custom-dtype", "fp32", "--prompt-token-ids", ",".join(map(str, prompt)), "--max-new-tokens", "5",
                           "--repeats", "2", "--block-size", str(page)]) == 0
    printed = capsys.readouterr().out
    assert f"Response: {plain.greedy_generate(config, tensors, prompt, 5)}" in printed
    assert "Prompt tokens: 7 | Generated tokens: 5" in printed and "Time to first token:" in printed and "median decode throughput:" in printed
    assert benchmark.main(["--model", folder, "--prompt", "text without a tokenizer"]) == 2
    assert benchmark.main(["--random-config", "tiny-b", "--mixed-requests", "6", "--mixed-prompt-range", "4,40", "--shared-prefix-tokens", "16",
                           "--output-tokens", "5", "--block-size", "8", "--max-num-batched-tokens", "64", "--profile",
                           "--profile-out", str(tmp_path / "kernels.txt")]) == 0
    printed = capsys.readouterr().out
    assert "mixed: 6 requests" in printed and "step profile:" in printed and "decode_by_rows" in printed
    tables = (tmp_path / "kernels.txt").read_text()
    assert "decode batch=1 graphs=True" in tables and "decode batch=6 graphs=False" in tables and "prefill prompt=40" in tables
    assert "paged_attention" in tables and "gemm_skinny" in tables           # this repository's kernels, by name, with their times
