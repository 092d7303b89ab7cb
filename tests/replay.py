"""Helpers that cut requests into steps in several ways and compare the engine's logits
with the plain implementation's whole-sequence logits at the same positions."""
from __future__ import annotations

import random

import torch

import plain_qwen3 as plain
from arle_amd.engine import StepEntry


def plain_logits(cfg, weights, tokens):
    """float64 logits [T, V] of one whole sequence from the plain implementation."""
    return plain.forward_logits(weights, cfg, tokens, dtype=torch.float64)


def run_steps(engine, steps):
    """steps: list of {"entries": [(id, tokens, want)], "end": [ids]}.
    Returns {(id, position): float32 logits row (CPU)}."""
    got = {}
    for st in steps:
        entries, where = [], []
        for rid, toks, want in st["entries"]:
            if not engine.cache.is_live(rid):
                engine.add_request(rid)
            start = engine.length(rid)
            entries.append(StepEntry(rid, list(toks), list(want)))
            where.extend((rid, start + w) for w in want)
        if entries:
            logits = engine.step(entries).float().cpu()
            assert logits.shape[0] == len(where)
            for row, key in zip(logits, where):
                assert key not in got, f"position {key} produced twice"
                got[key] = row
        for rid in st.get("end", []):
            engine.end_request(rid)
        engine.cache.check()
    return got


def whole(rid, toks):
    return [{"entries": [(rid, toks, list(range(len(toks))))], "end": [rid]}]


def prefill_then_decode(rid, toks, tail=32):
    tail = min(tail, len(toks) - 1)
    head = len(toks) - tail
    steps = [{"entries": [(rid, toks[:head], list(range(head)))], "end": []}]
    for i in range(head, len(toks)):
        steps.append({"entries": [(rid, toks[i:i + 1], [0])], "end": []})
    steps[-1]["end"] = [rid]
    return steps


def portions(rid, toks, sizes=(5, 2, 7, 3, 16, 2, 9, 4, 13, 2)):
    steps, i, k = [], 0, 0
    while i < len(toks):
        n = min(sizes[k % len(sizes)], len(toks) - i)
        if len(toks) - i - n == 1:  # never leave a lone last token out of a portion of >= 2
            n += 1
        steps.append({"entries": [(rid, toks[i:i + n], list(range(n)))], "end": []})
        i += n
        k += 1
    steps[-1]["end"] = [rid]
    return steps


def mixed(requests: dict, max_live=4, seed=0, decode_tail=6, max_portion=9):
    """Up to `max_live` requests at a time; portions of some beside single tokens of others;
    a request may sit a step out; finished requests end and the next one is admitted."""
    rng = random.Random(seed)
    waiting = list(requests)
    live, done_at = [], {}
    fed = {r: 0 for r in requests}
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live:
            live.append(waiting.pop(0))
        entries, ends = [], []
        for rid in list(live):
            toks = requests[rid]
            left = len(toks) - fed[rid]
            if len(live) > 1 and rng.random() < 0.2:
                continue  # sits this step out
            if left <= decode_tail:
                n = 1
            else:
                n = min(rng.randint(2, max_portion), left - decode_tail)
                if n < 2:
                    n = min(2, left)
            entries.append((rid, toks[fed[rid]:fed[rid] + n], list(range(n))))
            fed[rid] += n
            if fed[rid] == len(toks):
                ends.append(rid)
                live.remove(rid)
        if entries:
            steps.append({"entries": entries, "end": ends})
    return steps


def compare(got, cfg, weights, requests, rel_tol, what=""):
    """max |engine - plain| over all rows, relative to the largest plain logit, must be <= rel_tol."""
    worst = (0.0, None)
    for rid, toks in requests.items():
        ref = plain_logits(cfg, weights, toks)
        scale = float(ref.abs().max())
        for p in range(len(toks)):
            assert (rid, p) in got, f"{what}: no logits for request {rid!r} position {p}"
            row = got[(rid, p)].double()
            assert torch.isfinite(row).all(), f"{what}: non-finite logits at {rid!r}:{p}"
            err = float((row - ref[p]).abs().max()) / scale
            if err > worst[0]:
                worst = (err, (rid, p))
    assert worst[0] <= rel_tol, (f"{what}: first/worst mismatch at request,position={worst[1]}: "
                                 f"relative error {worst[0]:.3e} > {rel_tol:.1e}")
    return worst[0]
