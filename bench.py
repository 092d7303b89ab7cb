"""Decode and prefill throughput of the Qwen3-4B shape with random weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--layers L]

A step is one decode step of `batch` requests, each holding a `prompt`-token random prompt
(prefilled by the engine itself before the clock starts) and growing by one token per step.
`value` is decoded tokens per second over exactly K timed steps.  The same line carries the
prefill of one 2,048-token prompt, the decode step's HBM roofline, and decode at batch 1 and 64.
"""
from __future__ import annotations

import argparse
import json
import sys
import time

PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

# BASELINE.json configs[2]: Qwen3-4B shape
QWEN3_4B = dict(num_hidden_layers=36, hidden_size=2560, num_attention_heads=32, num_key_value_heads=8,
                head_dim=128, intermediate_size=9728, vocab_size=151936, rope_theta=1000000.0,
                rms_norm_eps=1e-6, tie_word_embeddings=True, max_position_embeddings=40960)
FULL_LAYERS = QWEN3_4B["num_hidden_layers"]
CONTEXT = 4096
PROMPT = 2048
PAGE = 16


def layer_params(c) -> int:
    q, kv = c["num_attention_heads"] * c["head_dim"], c["num_key_value_heads"] * c["head_dim"]
    h, i = c["hidden_size"], c["intermediate_size"]
    return h * (q + 2 * kv) + q * h + 3 * h * i


def decode_bytes(c, batch: int, context: float, elt: int = 2) -> float:
    """Bytes one decode step has to read: every weight once and the cache of the live requests."""
    L, h = c["num_hidden_layers"], c["hidden_size"]
    weights = (L * (layer_params(c) + 2 * h + 2 * c["head_dim"]) + h + c["vocab_size"] * h) * elt
    kv = batch * context * 2 * L * c["num_key_value_heads"] * c["head_dim"] * elt
    return weights + kv


def prefill_flops(c, tokens: int) -> float:
    L = c["num_hidden_layers"]
    gemm = 2.0 * tokens * L * layer_params(c)
    attn = 4.0 * c["num_attention_heads"] * c["head_dim"] * (tokens * (tokens + 1) / 2) * L
    head = 2.0 * c["vocab_size"] * c["hidden_size"]
    return gemm + attn + head


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=FULL_LAYERS)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 decode points")
    ap.add_argument("--prefill-only", action="store_true",
                    help="measure the 2,048-token prefill alone (for profiles of its kernels) and print that")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this engine has no multi-GPU path (asked for --gpus {args.gpus})")
        return 2

    import torch

    from arle_amd.config import Qwen3Config
    from arle_amd.engine import Engine, StepEntry
    from arle_amd.kernels import ops

    raw = dict(QWEN3_4B, num_hidden_layers=args.layers)
    config = Qwen3Config.from_dict(raw)
    dkey = "bf16" if args.dtype == "bfloat16" else "fp32"
    elt = 2 if dkey == "bf16" else 4
    max_batch = args.batch if args.no_points else max(args.batch, 64)
    t0 = time.time()
    engine = Engine.from_config("Qwen3ForCausalLM", config, seed=0, std=0.02, dtype=args.dtype,
                                page_size=PAGE, max_tokens=max_batch * CONTEXT, max_slots=max_batch,
                                max_request_tokens=CONTEXT)
    print(f"[bench] engine ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    gen = torch.Generator().manual_seed(1234)

    def prompt_tokens(n):
        return torch.randint(0, config.vocab_size, (n,), generator=gen).tolist()

    def timed(fn):
        torch.cuda.synchronize()
        t = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        return time.perf_counter() - t

    # ---- prefill: one 2,048-token prompt, logits of its last token included -----------------
    def prefill_once(key):
        engine.add_request(key)
        toks = prompt_tokens(PROMPT)
        dt = timed(lambda: ops.argmax_rows(engine.step([StepEntry(key, toks, [PROMPT - 1])])))
        engine.end_request(key)
        return dt

    for i in range(2):
        prefill_once(("warm", i))
    prefill_s = min(prefill_once(("prefill", i)) for i in range(3))
    prefill = {"value": round(PROMPT / prefill_s, 1), "tokens": PROMPT, "ms": round(prefill_s * 1e3, 3),
               "frac": round(prefill_flops(raw, PROMPT) / prefill_s / PEAK_FLOPS[dkey], 4)}
    print(f"[bench] prefill {prefill}", file=sys.stderr, flush=True)
    if args.prefill_only:
        print(json.dumps({"metric": "prefill tok/s at 2,048 tokens (Qwen3-4B shape, random weights)",
                          "value": prefill["value"], "unit": "tok/s", "n_gpus": 1, "dtype": dkey,
                          "higher_is_better": True, "prefill": prefill}))
        return 0

    # ---- decode ---------------------------------------------------------------------------------
    def decode_run(batch, steps, warmup):
        keys = [("d", batch, i) for i in range(batch)]
        last = []
        for k in keys:
            engine.add_request(k)
        per_step = max(1, 8192 // PROMPT)
        for i in range(0, batch, per_step):   # real prefill of every request, a few prompts a step
            group = keys[i:i + per_step]
            out = engine.step([StepEntry(k, prompt_tokens(PROMPT), [PROMPT - 1]) for k in group])
            last.extend(ops.argmax_rows(out).tolist())
        state = {"last": last}

        def one_step():
            out = engine.step([StepEntry(k, [t], [0]) for k, t in zip(keys, state["last"])])
            state["last"] = ops.argmax_rows(out).tolist()   # the host needs the token to go on

        for _ in range(warmup):
            one_step()
        ctx0 = engine.length(keys[0])
        dt = timed(lambda: [one_step() for _ in range(steps)])
        ctx_mean = ctx0 + (steps - 1) / 2.0 + 1
        for k in keys:
            engine.end_request(k)
        return dt, ctx_mean

    dt, ctx_mean = decode_run(args.batch, args.steps, args.warmup)
    ms_per_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    achieved = decode_bytes(raw, args.batch, ctx_mean, elt) / (dt / args.steps) / 1e9
    print(f"[bench] decode b{args.batch}: {value:.1f} tok/s, {ms_per_step:.3f} ms/step", file=sys.stderr, flush=True)
    points = {}
    if not args.no_points:
        for b in (1, 64):
            steps = min(args.steps, 32) if b == 64 else args.steps
            d, _ = decode_run(b, steps, max(2, args.warmup // 2))
            points[f"decode_b{b}"] = round(b * steps / d, 1)
            print(f"[bench] decode b{b}: {points[f'decode_b{b}']} tok/s", file=sys.stderr, flush=True)

    line = {
        "metric": "decode tok/s at batch 8, 2,048-token prompts (Qwen3-4B shape, random weights)",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dkey, "data": "synthetic: seeded random weights N(0,0.02), uniform random token ids",
        "config": {"model": "Qwen3-4B shape", "global_batch": args.batch, "seq_len": CONTEXT, "prompt_len": PROMPT,
                   "parallelism": "single GPU", "layers": args.layers, "layers_full": FULL_LAYERS,
                   "hidden": raw["hidden_size"], "q_heads": raw["num_attention_heads"],
                   "kv_heads": raw["num_key_value_heads"], "head_dim": raw["head_dim"],
                   "intermediate": raw["intermediate_size"], "vocab": raw["vocab_size"],
                   "rope_theta": raw["rope_theta"], "rms_norm_eps": raw["rms_norm_eps"], "tied": True,
                   "page_size": PAGE},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4)},
        "points": points,
    }
    if args.batch != 8:
        line["metric"] = line["metric"].replace("batch 8", f"batch {args.batch}")
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
