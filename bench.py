"""Decode and prefill throughput of the Qwen3-4B shape with random weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--layers L]
    python bench.py --workload qwen3-8b-mixed | qwen3-32b-decode     (two further workloads)

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

# the benchmark configuration: Qwen3-4B shape
QWEN3_4B = dict(num_hidden_layers=36, hidden_size=2560, num_attention_heads=32, num_key_value_heads=8,
                head_dim=128, intermediate_size=9728, vocab_size=151936, rope_theta=1000000.0,
                rms_norm_eps=1e-6, tie_word_embeddings=True, max_position_embeddings=40960)
# the two further workloads (`--workload`): Qwen3-8B and Qwen3-32B shapes
QWEN3_8B = dict(num_hidden_layers=36, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8,
                head_dim=128, intermediate_size=12288, vocab_size=151936, rope_theta=1000000.0,
                rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=40960)
QWEN3_32B = dict(num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, num_key_value_heads=8,
                 head_dim=128, intermediate_size=25600, vocab_size=151936, rope_theta=1000000.0,
                 rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=40960)
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


def _timed(torch, fn):
    torch.cuda.synchronize()
    t = time.perf_counter()
    fn()
    torch.cuda.synchronize()
    return time.perf_counter() - t


def ceilings() -> int:
    """What a kernel that only reads memory and one that only multiplies reach on this GPU, against the published peaks."""
    from arle_amd.kernels import ceilings as c

    read = c.read_bandwidth()
    small = c.read_bandwidth(launches=40)
    m32, m16 = c.mfma_rate(shape=32), c.mfma_rate(shape=16)
    print(json.dumps({
        "metric": "measured ceilings of one GPU", "unit": "GB/s and TFLOP/s",
        "hbm_read_gbs": round(read["best"] / 1e9, 1), "hbm_read_frac_of_peak": round(read["best"] / 1e9 / PEAK_HBM_GBS, 4),
        "hbm_read_100mb_launches_gbs": round(small["best"] / 1e9, 1),
        "hbm_read_by_workgroups_gbs": {str(k): round(v / 1e9, 1) for k, v in read["by_workgroups"].items()},
        "mfma_bf16_32x32x16_tflops": round(m32 / 1e12, 1), "mfma_bf16_16x16x32_tflops": round(m16 / 1e12, 1),
        "mfma_frac_of_peak": round(max(m32, m16) / PEAK_FLOPS["bf16"], 4)}))
    return 0


def mixed_8b(args) -> int:
    """Qwen3-8B shape: 32 requests decoding at 1,024 tokens of context beside one 2,048-token prompt
    that arrives in portions of 512: four steps of 32 + 512 rows.  Reports the mean step and the tokens a second
    of both kinds."""
    import torch

    from arle_amd.config import Qwen3Config
    from arle_amd.engine import Engine, StepEntry
    from arle_amd.kernels import ops

    raw = dict(QWEN3_8B, num_hidden_layers=args.layers or QWEN3_8B["num_hidden_layers"])
    config = Qwen3Config.from_dict(raw)
    decoders, context, prompt, portion = 32, 1024, 2048, 512
    engine = Engine.from_config("Qwen3ForCausalLM", config, seed=0, std=0.02, dtype="bfloat16", page_size=PAGE,
                                max_tokens=decoders * (context + 64) + 2 * prompt, max_slots=decoders + 1,
                                max_request_tokens=4096)
    gen = torch.Generator().manual_seed(1234)
    rand = lambda n: torch.randint(0, config.vocab_size, (n,), generator=gen).tolist()
    keys = [("d", i) for i in range(decoders)]
    last = []
    for k in keys:
        engine.add_request(k)
    for i in range(0, decoders, 8):
        out = engine.step([StepEntry(k, rand(context - 1), [context - 2]) for k in keys[i:i + 8]])
        last.extend(ops.argmax_rows(out).tolist())
    state = {"last": last}

    def one_prompt(tag):
        engine.add_request(tag)
        toks = rand(prompt)
        for a in range(0, prompt, portion):
            entries = [StepEntry(k, [t], [0]) for k, t in zip(keys, state["last"])]
            entries.append(StepEntry(tag, toks[a:a + portion], [portion - 1] if a + portion == prompt else []))
            out = engine.step(entries)
            state["last"] = ops.argmax_rows(out).tolist()[:decoders]
        engine.end_request(tag)

    for i in range(2):          # the second pass captures the four step shapes, later ones replay them
        one_prompt(("warm", i))
    # the decoders have grown by 8 tokens; the timed prompts run at 1,032..1,048 tokens of context
    reps = max(1, args.steps // 4)
    dt = _timed(torch, lambda: [one_prompt(("p", i)) for i in range(reps)])
    steps = 4 * reps
    ms = dt / steps * 1e3
    flops = sum(prefill_flops_portion(raw, a, portion) for a in range(0, prompt, portion)) / 4.0
    line = {"metric": "mixed step: 32 decoding requests at 1,024 tokens + a 512-token prompt portion (Qwen3-8B shape)",
            "value": round(steps * (decoders + portion) / dt, 1), "unit": "tok/s", "n_gpus": 1, "steps": steps,
            "warmup": 8, "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16", "data": "synthetic: seeded random weights N(0,0.02), uniform random token ids",
            "config": {"model": "Qwen3-8B shape", "decoding_requests": decoders, "decode_context": context,
                       "prompt_len": prompt, "portion": portion, "layers": raw["num_hidden_layers"],
                       "hidden": raw["hidden_size"], "q_heads": 32, "kv_heads": 8, "head_dim": 128,
                       "intermediate": raw["intermediate_size"], "vocab": raw["vocab_size"], "tied": False,
                       "page_size": PAGE},
            "points": {"decode_tok_s": round(decoders * steps / dt, 1), "prefill_tok_s": round(portion * steps / dt, 1)},
            "roofline": {"bound": "mfma+hbm", "flops_per_step": round(flops / 1e12, 2), "unit": "TFLOP",
                         "frac": round(flops / (dt / steps) / PEAK_FLOPS["bf16"], 4)}}
    print(json.dumps(line))
    return 0


def prefill_flops_portion(c, start: int, n: int) -> float:
    """Flops of a portion of n prompt tokens that starts at position `start` (products and causal attention)."""
    L = c["num_hidden_layers"]
    gemm = 2.0 * n * L * layer_params(c)
    attn = 4.0 * c["num_attention_heads"] * c["head_dim"] * (n * start + n * (n + 1) / 2) * L
    return gemm + attn


def decode_32b(args) -> int:
    """Qwen3-32B shape: 64 requests decoding at 8,192 tokens of context by default (65 GB of
    weights, 137 GB of cache)."""
    import torch

    from arle_amd.config import Qwen3Config
    from arle_amd.engine import Engine, StepEntry
    from arle_amd.kernels import ops

    raw = dict(QWEN3_32B, num_hidden_layers=args.layers or QWEN3_32B["num_hidden_layers"])
    config = Qwen3Config.from_dict(raw)
    batch, context = args.batch or 64, args.context
    steps, warmup = min(args.steps, 16), min(args.warmup, 4)
    t0 = time.time()
    engine = Engine.from_config("Qwen3ForCausalLM", config, seed=0, std=0.02, dtype="bfloat16", page_size=PAGE,
                                max_tokens=batch * (context + 64), max_slots=batch, max_request_tokens=context + 64)
    print(f"[bench] engine ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    gen = torch.Generator().manual_seed(1234)
    rand = lambda n: torch.randint(0, config.vocab_size, (n,), generator=gen).tolist()
    keys = [("d", i) for i in range(batch)]
    last = []
    for i, k in enumerate(keys):          # real prefill, one 8,191-token prompt a step
        engine.add_request(k)
        out = engine.step([StepEntry(k, rand(context - 1), [context - 2])])
        last.extend(ops.argmax_rows(out).tolist())
        if i % 8 == 7:
            print(f"[bench] prefilled {i + 1} of {batch} requests ({time.time() - t0:.0f} s)", file=sys.stderr, flush=True)
    state = {"last": last}

    def one_step():
        out = engine.step([StepEntry(k, [t], [0]) for k, t in zip(keys, state["last"])])
        state["last"] = ops.argmax_rows(out).tolist()

    for _ in range(warmup):
        one_step()
    ctx0 = engine.length(keys[0])
    dt = _timed(torch, lambda: [one_step() for _ in range(steps)])
    ctx_mean = ctx0 + (steps - 1) / 2.0 + 1
    achieved = decode_bytes(raw, batch, ctx_mean) / (dt / steps) / 1e9
    line = {"metric": f"decode tok/s at batch {batch}, {context:,} tokens of context (Qwen3-32B shape, random weights)",
            "value": round(batch * steps / dt, 1), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
            "ms_per_step": round(dt / steps * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16", "data": "synthetic: seeded random weights N(0,0.02), uniform random token ids",
            "config": {"model": "Qwen3-32B shape", "global_batch": batch, "seq_len": context, "layers": raw["num_hidden_layers"],
                       "layers_full": QWEN3_32B["num_hidden_layers"], "hidden": raw["hidden_size"], "q_heads": 64,
                       "kv_heads": 8, "head_dim": 128, "intermediate": raw["intermediate_size"],
                       "vocab": raw["vocab_size"], "tied": False, "page_size": PAGE},
            "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                         "frac": round(achieved / PEAK_HBM_GBS, 4)}}
    print(json.dumps(line))
    return 0


def main() -> int:
    global PAGE
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=None, help="decoding requests (default: 8; 64 for qwen3-32b-decode)")
    ap.add_argument("--context", type=int, default=8192, help="tokens of context of the qwen3-32b-decode workload")
    ap.add_argument("--layers", type=int, default=FULL_LAYERS)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--page-size", type=int, default=PAGE, help="tokens per cache page")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 decode points")
    ap.add_argument("--no-weight-tiles", action="store_true",
                    help="without the second copy of the projection weights that the few-rows kernels stream")
    ap.add_argument("--ceilings", action="store_true",
                    help="measure what a kernel that only reads, and one that only multiplies, reach on this GPU, and exit")
    ap.add_argument("--prefill-only", action="store_true",
                    help="measure the 2,048-token prefill alone (for profiles of its kernels) and print that")
    ap.add_argument("--workload", default="qwen3-4b", choices=["qwen3-4b", "qwen3-8b-mixed", "qwen3-32b-decode"],
                    help="qwen3-4b is the default run; the other two are further workloads at larger shapes")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this engine has no multi-GPU path (asked for --gpus {args.gpus})")
        return 2
    PAGE = args.page_size
    if args.ceilings:
        return ceilings()
    if args.workload == "qwen3-4b" and args.batch is None:
        args.batch = 8
    if args.workload != "qwen3-4b":
        if args.layers == FULL_LAYERS:
            args.layers = 0   # the workload's own depth
        return mixed_8b(args) if args.workload == "qwen3-8b-mixed" else decode_32b(args)

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
                                max_request_tokens=CONTEXT, weight_tiles=False if args.no_weight_tiles else None)
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
                   "page_size": PAGE, "weight_tiles": engine.rt.weight_tiles},
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
