"""Traces for the replay program: the same requests cut into steps in different ways.

A trace is a list of step records in the replay program's JSON format.  Every step asks for the
logits of all the tokens it feeds, so that every position of every request can be compared with
the plain implementation, whatever the cut.
"""
from __future__ import annotations

import json
import os
import random
from typing import Dict, List, Sequence, Tuple

import numpy as np


def round64(n: int) -> int:
    return -(-n // 64) * 64


def _entry(rid, tokens, start, end):
    return {"id": rid, "tokens": list(tokens[start:end]), "want": list(range(end - start))}


def whole(requests: Dict[str, Sequence[int]]) -> List[dict]:
    """Each request alone and whole, one after the other."""
    return [{"step": i, "entries": [_entry(rid, tokens, 0, len(tokens))], "end": [rid]}
            for i, (rid, tokens) in enumerate(requests.items())]


def tail_decoded(requests, tail: int = 32) -> List[dict]:
    """Most of a request in one step, its last ``tail`` tokens one by one."""
    steps = []
    for rid, tokens in requests.items():
        head = max(1, len(tokens) - tail)
        cuts = [(0, head)] + [(p, p + 1) for p in range(head, len(tokens))]
        for start, end in cuts:
            steps.append({"step": len(steps), "entries": [_entry(rid, tokens, start, end)],
                          "end": [rid] if end == len(tokens) else []})
    return steps


def changing_portions(requests, sizes=(7, 2, 33, 3, 16, 2, 5, 64, 2, 17)) -> List[dict]:
    """Portions of changing size, down to two tokens."""
    steps = []
    for rid, tokens in requests.items():
        start, turn = 0, 0
        while start < len(tokens):
            end = min(len(tokens), start + sizes[turn % len(sizes)])
            if len(tokens) - end == 1:          # do not leave a single token: keep the smallest portion at two
                end = len(tokens)
            steps.append({"step": len(steps), "entries": [_entry(rid, tokens, start, end)],
                          "end": [rid] if end == len(tokens) else []})
            start, turn = end, turn + 1
    return steps


def mixed(requests, seed: int, budget_tokens: int, max_live: int = 4, decode_tail: int = 6) -> List[dict]:
    """Up to ``max_live`` requests at a time, portions of some beside single tokens of others,
    requests left out of steps now and then, under a token budget so small that the pages of
    finished requests are used again by later ones."""
    rng = random.Random(seed)
    waiting = list(requests.items())
    live: List[Tuple[str, Sequence[int]]] = []
    done_upto: Dict[str, int] = {}
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live and sum(round64(len(t)) for _, t in live) + round64(len(waiting[0][1])) <= budget_tokens:
            rid, tokens = waiting.pop(0)
            live.append((rid, tokens))
            done_upto[rid] = 0
        if not live:
            raise ValueError("budget_tokens is too small for the next request")
        entries, ended = [], []
        for rid, tokens in live:
            if len(live) > 1 and rng.random() < 0.25:
                continue                              # left out of this step, goes on later
            start = done_upto[rid]
            remaining = len(tokens) - start
            size = 1 if remaining <= decode_tail else rng.choice((2, 3, 5, 16, 31, 40))
            end = min(len(tokens), start + size)
            entries.append(_entry(rid, tokens, start, end))
            done_upto[rid] = end
            if end == len(tokens):
                ended.append(rid)
        if not entries:
            continue
        steps.append({"step": len(steps), "entries": entries, "end": ended})
        live = [(rid, tokens) for rid, tokens in live if rid not in ended]
    return steps


def peak_tokens(steps) -> int:
    """Most tokens live requests hold at any time, each rounded up to a multiple of 64."""
    held, peak = {}, 0
    for step in steps:
        for entry in step["entries"]:
            held[entry["id"]] = held.get(entry["id"], 0) + len(entry["tokens"])
        peak = max(peak, sum(round64(n) for n in held.values()))
        for rid in step["end"]:
            held.pop(rid, None)
    return peak


def to_lines(steps) -> str:
    return "".join(json.dumps(step) + "\n" for step in steps)


def collect(steps, out_dir: str, vocab: int) -> Dict[Tuple[str, int], np.ndarray]:
    """(request, position) -> logits, read back from the files the replay wrote."""
    results, position = {}, {}
    for step in steps:
        wanted = sum(len(entry["want"]) for entry in step["entries"])
        rows = None
        if wanted:
            rows = np.fromfile(os.path.join(out_dir, f"{step['step']}.f32"), dtype="<f4").reshape(wanted, vocab)
        row = 0
        for entry in step["entries"]:
            start = position.get(entry["id"], 0)
            for place in entry["want"]:
                results[(entry["id"], start + place)] = rows[row]
                row += 1
            position[entry["id"]] = start + len(entry["tokens"])
    return results
