"""bin/trace_run on the GPU, as a user runs it: the same requests whole, with the last 32 tokens
decoded one by one, in portions of changing size, and mixed with other requests so that pages are
used again; in float32 and in bfloat16; every position against the plain implementation."""
import os
import subprocess
import sys

import numpy as np
import pytest

import traces
from helpers import check_against_rounded_oracle, model_folder, plain_logits, random_tokens, relative_error, rounded_logits
from tiny_configs import CASES

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
pytestmark = pytest.mark.gpu

TOLERANCE = {"float32": dict(atol=3e-5, rtol=1e-4), "bfloat16": None}
# bfloat16 keeps 8 bits, and a few roundings of that size meet through two or three layers.  The error of a position's
# logits is measured against those logits' own size (their largest magnitude; the tiny models' logits are a few tenths,
# so an absolute bound would hide a wrong key or page), and held against what the plain implementation loses on the same
# sequences when it rounds to bfloat16 where the reference's kernels round (helpers.check_against_rounded_oracle).


def rounded_errors(case, lengths_and_seeds):
    """Per position, what the rounded oracle loses on these sequences."""
    return [relative_error(row, exact) for n, seed in lengths_and_seeds
            for row, exact in zip(rounded_logits(case, n, seed).numpy(), plain_logits(case, n, seed).numpy())]


def build_trace(case):
    vocab = CASES[case][0]["vocab_size"]
    lengths = {"a": 70, "b": 33, "c": 100}
    mixed_lengths = (5, 17, 33, 70, 100, 41, 64, 1, 90, 130, 20, 77)
    meta, steps = {}, []

    def add(prefix, requests_meta, maker):
        requests = {f"{prefix}{rid}": random_tokens(vocab, n, seed) for rid, (n, seed) in requests_meta.items()}
        meta.update({f"{prefix}{rid}": v for rid, v in requests_meta.items()})
        part = maker(requests)
        for step in part:
            step["step"] = len(steps)
            steps.append(step)
        return part

    base = {rid: (n, 100 + i) for i, (rid, n) in enumerate(lengths.items())}
    add("w-", base, traces.whole)
    add("t-", base, lambda r: traces.tail_decoded(r, 32))
    add("p-", base, traces.changing_portions)
    mixed = add("m-", {f"q{i}": (n, 200 + i) for i, n in enumerate(mixed_lengths)}, lambda r: traces.mixed(r, seed=7, budget_tokens=256))
    assert max(len(s["entries"]) for s in mixed) >= 3
    return steps, meta


def run_trace(case, dtype, steps, tmp_path, max_tokens, page_size):
    out = tmp_path / f"out-{case}-{dtype}"
    command = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_folder(case), "--dtype", dtype,
               "--out", str(out), "--max-tokens", str(max_tokens), "--page-size", str(page_size)]
    done = subprocess.run(command, input=traces.to_lines(steps), capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-3000:]
    assert done.stdout.split() == [w for s in steps for w in ("done", str(s["step"]))]
    return traces.collect(steps, str(out), CASES[case][0]["vocab_size"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("case, page_size", [("A", 16), ("B", 8), ("C", 4), ("D", 16)])
def test_all_schedules_match_the_plain_implementation(case, page_size, dtype, tmp_path):
    print(f"replay case {case} {dtype} page {page_size}", flush=True)
    steps, meta = build_trace(case)
    max_tokens = traces.peak_tokens(steps)
    assert max_tokens <= 256
    results = run_trace(case, dtype, steps, tmp_path, max_tokens, page_size)
    assert len(results) == sum(n for n, _ in meta.values())
    errors = []
    for (rid, position), logits in results.items():
        n, seed = meta[rid]
        expected = plain_logits(case, n, seed)[position].numpy()
        if dtype == "float32":
            np.testing.assert_allclose(logits, expected, err_msg=f"{rid} position {position}", **TOLERANCE["float32"])
        else:
            errors.append(relative_error(logits, expected))
    lost = rounded_errors(case, sorted(set(meta.values()))) if errors else None
    if errors:
        check_against_rounded_oracle(errors, lost, f"case {case} against the plain implementation")
    # the same request cut differently agrees with itself at least as well as with the oracle
    errors = []
    for rid in ("a", "b", "c"):
        n, _ = meta[f"w-{rid}"]
        for position in range(n):
            for other in ("t-", "p-"):
                a, b = results[(f"w-{rid}", position)], results[(f"{other}{rid}", position)]
                if dtype == "float32":
                    assert float(np.abs(a - b).max()) <= 1e-4, (rid, other, position)
                else:
                    errors.append(relative_error(b, a))
    if errors:      # two runs that each lose what the rounded oracle loses differ by about 1.4 times that
        check_against_rounded_oracle(errors, lost, f"case {case} between two cuts of the same request", factor=2.0)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_first_tokens(dtype, tmp_path):
    """A one-token prompt decoded for 300 tokens, crossing many pages; and the very first positions."""
    case = "B"
    vocab = CASES[case][0]["vocab_size"]
    tokens = random_tokens(vocab, 301, 31)
    steps = traces.tail_decoded({"long": tokens}, tail=300)
    assert len(steps) == 301 and all(len(s["entries"][0]["tokens"]) == 1 for s in steps)
    results = run_trace(case, dtype, steps, tmp_path, 320, 8)
    expected = plain_logits(case, 301, 31).numpy()
    errors = []
    for position in range(301):
        got = results[("long", position)]
        if dtype == "float32":
            np.testing.assert_allclose(got, expected[position], err_msg=f"position {position}", **TOLERANCE["float32"])
        else:
            errors.append(relative_error(got, expected[position]))
    if errors:
        check_against_rounded_oracle(errors, rounded_errors(case, [(301, 31)]), "long decoding")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unusual_steps(dtype, tmp_path):
    """Wanted places out of order and twice; a step with nothing in it; a first token alone; five live requests; a
    request left out of steps; a name ended and used again for other tokens; an end of somebody unknown; a step
    that wants nothing (no file)."""
    import plain_qwen3 as plain
    from helpers import BF16, plain_model
    case = "B"
    vocab = CASES[case][0]["vocab_size"]
    config, tensors = plain_model(case)
    t = {k: random_tokens(vocab, n, 70 + i) for i, (k, n) in enumerate({"a": 64, "b": 1, "c": 30, "d": 64, "e": 17, "f": 5}.items())}
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": t["a"][:10], "want": [9, 0, 9, 3]}, {"id": "b", "tokens": t["b"], "want": [0]}], "end": ["b", "nobody"]},
        {"step": 1, "entries": [], "end": []},
        {"step": 2, "entries": [{"id": "c", "tokens": t["c"][:1], "want": [0]}], "end": []},
        {"step": 3, "entries": [{"id": "a", "tokens": t["a"][10:12], "want": []}, {"id": "c", "tokens": t["c"][1:2], "want": []}], "end": []},
        {"step": 4, "entries": [{"id": "c", "tokens": t["c"][2:3], "want": [0]}, {"id": "d", "tokens": t["d"][:1], "want": []},
                                {"id": "e", "tokens": t["e"][:1], "want": [0]}, {"id": "f", "tokens": t["f"][:1], "want": [0]},
                                {"id": "a", "tokens": t["a"][12:13], "want": [0]}], "end": ["f"]},
        {"step": 5, "entries": [{"id": "b", "tokens": t["c"][:7], "want": [6]}], "end": []},
        {"step": 6, "entries": [{"id": "a", "tokens": t["a"][13:64], "want": [50]}, {"id": "d", "tokens": t["d"][1:64], "want": [62, 0]}],
         "end": ["a", "d", "e", "b", "c"]},
        {"step": 7, "entries": [{"id": "a", "tokens": t["d"][:64], "want": [63]}], "end": ["a"]},
    ]
    out = tmp_path / "out"
    command = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_folder(case), "--dtype", dtype,
               "--out", str(out), "--max-tokens", str(5 * 64), "--page-size", "8"]
    done = subprocess.run(command, input=traces.to_lines(steps), capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-3000:]
    assert done.stdout.split() == [w for s in steps for w in ("done", str(s["step"]))]
    assert sorted(os.listdir(out)) == ["0.f32", "2.f32", "4.f32", "5.f32", "6.f32", "7.f32"]       # steps 1 and 3 want nothing
    fed, place, errors, lost, sequences = {}, {}, [], [], []
    for step in steps:
        wanted = sum(len(e["want"]) for e in step["entries"])
        rows = np.fromfile(out / f"{step['step']}.f32", dtype="<f4").reshape(wanted, vocab) if wanted else None
        row = 0
        for entry in step["entries"]:
            start = place.get(entry["id"], 0)
            fed.setdefault(entry["id"], []).extend(entry["tokens"])
            for want in entry["want"]:
                expected = plain.forward(config, tensors, fed[entry["id"]]).numpy()[start + want]
                if dtype == "float32":
                    np.testing.assert_allclose(rows[row], expected, err_msg=f"step {step['step']} {entry['id']} place {want}", **TOLERANCE["float32"])
                else:
                    errors.append(relative_error(rows[row], expected))
                row += 1
            place[entry["id"]] = start + len(entry["tokens"])
        for name in step["end"]:
            place.pop(name, None)
            sequences.append(fed.pop(name, None))
    if errors:      # a dozen places wanted: held against what the rounded oracle loses anywhere in these sequences
        for tokens in filter(None, sequences + list(fed.values())):
            lost.extend(relative_error(row, exact) for row, exact in zip(plain.forward(config, tensors, tokens, r=BF16).numpy(),
                                                                         plain.forward(config, tensors, tokens).numpy()))
        check_against_rounded_oracle(errors, lost, "unusual steps")


def test_two_bfloat16_runs_write_the_same_bytes(tmp_path):
    """Which kernel a shape goes through comes from a table, never from a stopwatch: a second process rounds as the first."""
    case = "D"
    vocab = CASES[case][0]["vocab_size"]
    requests = {"a": random_tokens(vocab, 90, 3), "b": random_tokens(vocab, 40, 4)}
    steps = traces.mixed(requests, seed=1, budget_tokens=192) + traces.tail_decoded({"c": random_tokens(vocab, 50, 5)}, 20)
    for index, step in enumerate(steps):
        step["step"] = index
    outs = []
    for run in range(2):
        (tmp_path / str(run)).mkdir()
        run_trace(case, "bfloat16", steps, tmp_path / str(run), 256, 16)
        folder = tmp_path / str(run) / f"out-{case}-bfloat16"
        outs.append({name: (folder / name).read_bytes() for name in sorted(os.listdir(folder))})
    assert outs[0].keys() == outs[1].keys() and len(outs[0]) > 10
    assert all(outs[0][name] == outs[1][name] for name in outs[0])
