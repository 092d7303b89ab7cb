"""Measure which kernel runs each matrix product of a model fastest, row count by row count, and write the table
that `ops.load_product_table` takes in.

The rules in `ops.product_by_rules` were measured at the widths of Qwen3-4B, 8B and 32B.  For other widths (or
another GPU) this module times every kernel that can run a shape (`ops.product_candidates`) against the others, with
weights that are cold (several copies taken in turn, more than the memory-side cache holds) and, for a product whose
result goes into a residual add and norm, with that kernel behind it, since a stack of partial products costs its
consumer what it saved the product.  The reference tunes its library products when its scheduler starts
(infer/src/scheduler/cuda/core/warmup.rs:100-131, `autotune_all_cached_gemms_cuda`); here the result is a file.
"""
from __future__ import annotations

import json
import time

import torch

from . import ops

ROWS = (1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 14, 16, 20, 24, 28, 32, 40, 48, 56, 64, 96, 128, 192, 256, 384, 512, 768, 1024, 1536,
        2048, 3072, 4096, 6144, 8192)
HEAD_ROWS = (1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 14, 16, 20, 24, 28, 32, 40, 48, 56, 64, 96, 128, 256)
COLD_BYTES = 600 << 20      # copies of a weight matrix taken in turn hold at least this much together


def model_products(hidden: int, q_width: int, kv_width: int, intermediate: int, vocab: int = 0) -> list:
    """(name, N, K, fused, consumer, row counts) of the products of a decoder: q|k|v, o, gate|up with its activation,
    down, and the output head if a vocabulary is given.  consumer "norm": the result goes into a residual add and
    norm (which can add a stack of partial products itself; the q/k/v preparation does the same); None: it is used
    as it is."""
    found = [("qkv", q_width + 2 * kv_width, hidden, False, "norm", ROWS), ("o", hidden, q_width, False, "norm", ROWS),
             ("gate_up", 2 * intermediate, hidden, True, None, ROWS), ("down", hidden, intermediate, False, "norm", ROWS)]
    if vocab:
        found.append(("head", vocab, hidden, False, None, HEAD_ROWS))
    return found


def _seconds(fn, iters: int, repeats: int = 3) -> float:
    """Seconds a call of fn takes on the GPU: `iters` calls are captured into one graph and the graph is replayed, so
    that the time is the kernels' and not the host's (a product of a few rows is shorter than its launch)."""
    for _ in range(2):
        fn()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(iters):
            fn()
    graph.replay()
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(repeats):
        start = time.perf_counter()
        graph.replay()
        torch.cuda.synchronize()
        best = min(best, (time.perf_counter() - start) / iters)
    return best


MIN_GAIN = 0.08     # a choice other than the rules' has to win by this much of the rule's time, and by MIN_GAIN_US
MIN_GAIN_US = 1.5   # (products timed alone gain a microsecond here and there that whole steps do not show)


def tune_products(products, device="cuda:0", tiled: bool = True, iters: int = 20, say=None, rows=None) -> tuple:
    """(table, report): table as `ops.load_product_table` reads it; report: one record a (product, row count) with
    the microseconds of every candidate, of the rules' choice and of the best.  products: (name, N, K, with the
    activation, consumer[, row counts]); rows: the row counts for all of them (default: each product's own, else
    ROWS)."""
    table, report = {}, []
    only = rows
    for name, n, k, fused, consumer, *own_rows in products:
        rows = only if only is not None else (own_rows[0] if own_rows else ROWS)
        copies = max(2, -(-COLD_BYTES // (n * k * 2)))
        weights = [torch.randn(n, k, device=device).mul_(0.02).to(torch.bfloat16) for _ in range(copies)]
        tiles = [ops.pack_weight_tiles(w) for w in weights] if tiled else [None] * copies
        norm_weight = torch.ones(n, dtype=torch.bfloat16, device=device)
        turn = {"i": 0}
        entries = []
        for m in rows:
            x = torch.randn(m, k, device=device).to(torch.bfloat16)
            residual = torch.zeros((m, n), dtype=torch.float32, device=device) if consumer == "norm" else None

            def run(choice):
                turn["i"] = (turn["i"] + 1) % copies
                y = ops.run_product(choice, x, weights[turn["i"]], tiles[turn["i"]], torch.bfloat16,
                                    partials_ok=consumer == "norm", fused=fused)
                if consumer == "norm":
                    ops.add_rmsnorm(residual, y, norm_weight, 1e-6, torch.bfloat16)

            ruled = ops.product_by_rules(m, n, k, k, tiled=tiled, fused=fused, partials_ok=consumer == "norm")
            timed = {}
            for choice in dict.fromkeys([ruled] + ops.product_candidates(m, n, k, k, tiled=tiled, fused=fused)):
                try:
                    timed[choice] = _seconds(lambda: run(choice), iters)
                except (ops.ShapeError, RuntimeError):
                    continue        # a kernel that refuses this shape is no candidate
            best = min(timed, key=timed.get)
            if timed[ruled] - timed[best] < max(MIN_GAIN * timed[ruled], MIN_GAIN_US * 1e-6):
                best = ruled        # what does not win clearly does not replace the rule
            entries.append([m, best.kernel, list(best.variant), best.splits])
            record = {"product": name, "rows": m, "rule": [ruled.kernel, list(ruled.variant), ruled.splits],
                      "rule_us": round(timed[ruled] * 1e6, 1), "best": [best.kernel, list(best.variant), best.splits],
                      "best_us": round(timed[best] * 1e6, 1),
                      "all_us": {f"{c.kernel}{list(c.variant)}/{c.splits}": round(t * 1e6, 1) for c, t in timed.items()}}
            report.append(record)
            if say is not None:
                say(record)
        # neighbouring row counts with one choice become one entry
        merged = []
        for entry in entries:
            if merged and merged[-1][1:] == entry[1:]:
                merged[-1][0] = entry[0]
            else:
                merged.append(list(entry))
        table[f"{n},{k},{int(fused)},{int(tiled)}"] = merged
        del weights, tiles
        torch.cuda.empty_cache()
    return table, report


def write_table(path: str, table: dict) -> None:
    with open(path, "w", encoding="utf-8") as fh:
        json.dump(table, fh, indent=1)
