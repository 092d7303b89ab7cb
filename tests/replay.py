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


# bfloat16 rows: beside the largest error of a row, its root-mean-square error over the vocabulary, relative to the
# root mean square of the plain row.  For random weights the two are of one size (a row's largest logit is about
# five times its rms, and so is its largest error), so the bound on it is no tighter than the maximum's; what it
# adds is the third check below.  Rounding makes every row of a comparison wrong by about the same amount: the
# rows went through the same layers and the same kernels.  A row whose rms error is several times the median of its
# comparison is not rounding, even where it stays under the absolute tolerances: one token's row of a product, one
# request's page, one head of one row.
RMS_TOL = {2e-2: 2.5e-2, 2.5e-2: 3e-2, 3e-2: 3e-2}
OUTLIER_TOL = 4.0     # measured over all comparisons of these tests: 1.1 to 3.0
last_stats: dict = {}


def row_errors(row: torch.Tensor, ref_row: torch.Tensor, scale: float):
    """(largest error / scale, rms error / rms of the plain row) of one row of logits."""
    diff = row.double() - ref_row.double()
    return float(diff.abs().max()) / scale, float(diff.pow(2).mean().sqrt() / ref_row.double().pow(2).mean().sqrt())


def check_rows(got, reference: dict, rel_tol, what="", rms_tol=None, need_all=True, outlier_tol=None):
    """got {(request, position): row} against reference {request: [T, V] plain logits}: the largest error of any
    row relative to the request's largest plain logit within rel_tol; every row's rms error within rms_tol
    (default: RMS_TOL[rel_tol] for the bfloat16 tolerances, none for float32's, whose maximum is tight already);
    and, with at least eight rows, no row's rms error more than outlier_tol times the median row's.
    Returns (worst maximum error, worst rms error)."""
    if rms_tol is None:
        rms_tol = RMS_TOL.get(rel_tol)
    if outlier_tol is None:
        outlier_tol = OUTLIER_TOL
    worst, worst_rms, every = (0.0, None), (0.0, None), []
    for rid, ref in reference.items():
        scale = float(ref.abs().max())
        for p in range(ref.shape[0]):
            if (rid, p) not in got:
                assert not need_all, f"{what}: no logits for request {rid!r} position {p}"
                continue
            row = got[(rid, p)]
            assert torch.isfinite(row).all(), f"{what}: non-finite logits at {rid!r}:{p}"
            err, rms = row_errors(row, ref[p], scale)
            every.append(rms)
            if err > worst[0]:
                worst = (err, (rid, p))
            if rms > worst_rms[0]:
                worst_rms = (rms, (rid, p))
    median = sorted(every)[len(every) // 2] if every else 0.0
    spread = worst_rms[0] / median if len(every) >= 8 and median > 0 else 0.0
    before = last_stats.get(what, (0.0, 0.0, 0.0))
    last_stats[what] = (max(before[0], worst[0]), max(before[1], worst_rms[0]), max(before[2], spread))
    assert worst[0] <= rel_tol, (f"{what}: first/worst mismatch at request,position={worst[1]}: "
                                 f"relative error {worst[0]:.3e} > {rel_tol:.1e}")
    if rms_tol is not None:
        assert worst_rms[0] <= rms_tol, (f"{what}: rms error of the row at request,position={worst_rms[1]}: "
                                         f"{worst_rms[0]:.3e} > {rms_tol:.1e}")
    assert spread <= outlier_tol, (f"{what}: the row at request,position={worst_rms[1]} is wrong by {spread:.1f} times "
                                   f"the median row's rms error ({worst_rms[0]:.3e} against {median:.3e})")
    return worst[0], worst_rms[0]


def compare(got, cfg, weights, requests, rel_tol, what="", rms_tol=None, outlier_tol=None):
    """Every row of every request against the plain implementation (see check_rows)."""
    reference = {rid: plain_logits(cfg, weights, toks) for rid, toks in requests.items()}
    return check_rows(got, reference, rel_tol, what, rms_tol, outlier_tol=outlier_tol)[0]
