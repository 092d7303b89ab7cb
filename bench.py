"""Decode and prefill throughput of the Qwen3-4B shape with random weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--layers L]
    python bench.py --workload qwen3-8b-mixed | qwen3-32b-decode     (two further workloads)
    python bench.py --generate                                       (the decode workload through LLM.generate)

A step is one decode step of `batch` requests, each holding a `prompt`-token random prompt
(prefilled by the engine itself before the clock starts) and growing by one token per step.
`value` is decoded tokens per second over exactly K timed steps.  The same line carries the
prefill of one 2,048-token prompt, the decode step's HBM roofline, and decode at batch 1 and 64.
"""
from __future__ import annotations

import argparse
import json
import os
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


# ---- where a step's time goes: kernels of a profiled step, sorted into the parts of a layer -------------------------

GEMM_NAMES = ("gemm_rows", "gemm_stream", "gemm_tiles", "gemm_f32", "Cijk_", "sum_partials", "silu_mul")
PARTS = ("qkv", "o", "gate_up", "down", "head", "attention", "qk_prep", "norm", "other")


def _template_args(name: str) -> list:
    return name[name.index("<") + 1:name.rindex(">")].replace(" ", "").split(",") if "<" in name and ">" in name else []


def _completes_gate_up(name: str) -> bool:
    """Whether this kernel leaves gate|up complete: a product with the activation fused (gemm_rows_kernel<MT, WN,
    WK, PD, XD, EPI, out> / gemm_tiles_kernel<MT, TN, PD, PX, PIPE, EPI, out> with EPI = 1), or the activation kernel
    behind a plain product."""
    if "silu_mul" in name:
        return True
    args = _template_args(name)
    if "gemm_rows_kernel" in name:
        return len(args) > 5 and args[5] == "1"
    if "gemm_tiles_kernel" in name:
        return len(args) > 5 and args[5] == "1"
    return False


def classify_step(names, layers: int) -> list:
    """The part of the model that each kernel of one step belongs to, from the order in which a layer launches
    them: norm, q|k|v product, q/k preparation (a kernel of its own, or inside the attention's for single decoded
    tokens), attention (+ merges), o product, norm, gate|up (+ activation), down product; after the last layer the
    final norm and the head."""
    out, phase, layers_done = [], "qkv", 0
    for name in names:
        if "qk_prep" in name:
            part, phase = "qk_prep", "o"
        elif "attn_" in name:
            part = "attention"
            if phase == "qkv":     # single decoded tokens: the attention's kernel prepares q, k and v itself
                phase = "o"
        elif "rmsnorm" in name:
            part = "norm"
            if phase == "o":
                phase = "gate_up"
            elif phase == "down":
                layers_done += 1
                phase = "head" if layers_done >= layers else "qkv"
        elif any(g in name for g in GEMM_NAMES):
            part = phase
            if phase == "gate_up" and _completes_gate_up(name):
                phase = "down"
        else:
            part = "other"
        out.append(part)
    return out


def profiled_steps(torch, fns) -> list:
    """The kernels of every call in `fns`, run one after the other inside ONE profiler session (a second session
    in a process has crashed the profiler here): a list, one entry a call, of (name, microseconds) in launch
    order.  A step begins with the embedding kernel, which is how the session's kernels are cut into calls."""
    from torch.profiler import ProfilerActivity, profile

    torch.cuda.synchronize()
    with profile(activities=[ProfilerActivity.CUDA]) as prof:
        for fn in fns:
            fn()
            torch.cuda.synchronize()
    evs = [e for e in prof.events() if e.device_type == torch.autograd.DeviceType.CUDA and "Memcpy" not in e.name
           and "Memset" not in e.name]
    evs.sort(key=lambda e: e.time_range.start)
    steps, early = [], []
    for e in evs:
        item = (e.name, e.time_range.end - e.time_range.start)
        if "embed_gather" in e.name:
            steps.append(early + [item])     # what ran before the first step's embedding is counted with it
            early = []
        elif steps:
            steps[-1].append(item)
        else:
            early.append(item)
    if len(steps) != len(fns):
        raise RuntimeError(f"the profiler saw {len(steps)} steps for {len(fns)} calls")
    return steps


def part_times(steps, layers: int) -> dict:
    """part -> microseconds a step (mean over `steps`, lists of (kernel name, microseconds)), plus "kernels".
    The profiler now and then loses kernels of a step; only the steps with the most kernels are counted, and
    those must show every layer."""
    most = max(len(k) for k in steps)
    steps = [k for k in steps if len(k) == most]
    for kernels in steps:
        seen = (sum(1 for n, _ in kernels if "rmsnorm" in n) - 1) // 2   # two norms a layer and the last one
        if seen != layers:
            raise RuntimeError(f"a profiled step shows {seen} of {layers} layers")
    total = {p: 0.0 for p in PARTS}
    for kernels in steps:
        for part, (_, us) in zip(classify_step([n for n, _ in kernels], layers), kernels):
            total[part] += us
    out = {p: t / len(steps) for p, t in total.items()}
    missing = [p for p in ("qkv", "o", "gate_up", "down", "head") if not out.get(p)]
    if missing:  # a kernel's name no longer says what the sorting reads from it
        raise RuntimeError(f"no kernel of a profiled step was sorted into {', '.join(missing)}")
    out["kernels"] = sum(len(k) for k in steps) / len(steps)
    return out


def part_bytes_decode(c, batch: int, context: float, elt: int = 2) -> dict:
    """Bytes that each part of a decode step has to read: its weights once, and for attention the cache."""
    L, h, i = c["num_hidden_layers"], c["hidden_size"], c["intermediate_size"]
    q, kv = c["num_attention_heads"] * c["head_dim"], c["num_key_value_heads"] * c["head_dim"]
    return {"qkv": L * h * (q + 2 * kv) * elt, "o": L * q * h * elt, "gate_up": L * 2 * i * h * elt,
            "down": L * h * i * elt, "head": c["vocab_size"] * h * elt, "attention": batch * context * 2 * L * kv * elt}


def part_flops_prefill(c, tokens: int) -> dict:
    L, h, i = c["num_hidden_layers"], c["hidden_size"], c["intermediate_size"]
    q, kv = c["num_attention_heads"] * c["head_dim"], c["num_key_value_heads"] * c["head_dim"]
    return {"qkv": 2.0 * tokens * L * h * (q + 2 * kv), "o": 2.0 * tokens * L * q * h,
            "gate_up": 2.0 * tokens * L * 2 * i * h, "down": 2.0 * tokens * L * h * i,
            "head": 2.0 * c["vocab_size"] * h, "attention": 4.0 * q * (tokens * (tokens + 1) / 2) * L}


def part_report(times: dict, work: dict, peak: float, ceiling: float) -> tuple:
    """(microseconds a step by part, fraction of the published peak, fraction of the measured ceiling)."""
    us = {p: round(times[p], 1) for p in PARTS if times.get(p)}
    us["kernels"] = round(times["kernels"], 1)
    of_peak = {p: round(work[p] / (times[p] * 1e-6) / peak, 4) for p in work if times.get(p)}
    of_ceiling = {p: round(work[p] / (times[p] * 1e-6) / ceiling, 4) for p in work if times.get(p)}
    return us, of_peak, of_ceiling


def parts_in_a_child_process(args) -> dict:
    """The breakdown by part of the model, measured by a second run of this program under the profiler: the
    profiler stays out of the process whose steps are timed, and a fault of its own costs only the breakdown."""
    import os
    import subprocess

    cmd = [sys.executable, os.path.abspath(__file__), "--parts-only", "--batch", str(args.batch), "--layers", str(args.layers),
           "--page-size", str(PAGE), "--dtype", args.dtype]
    cmd += ["--no-weight-tiles"] if args.no_weight_tiles else []
    try:
        res = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
        lines = [ln for ln in res.stdout.splitlines() if ln.startswith("{")]
        if res.returncode != 0 or not lines:
            return {"parts": f"not measured: the profiled run ended with code {res.returncode}"}
        return json.loads(lines[-1])
    except (subprocess.TimeoutExpired, OSError, ValueError) as exc:
        return {"parts": f"not measured: {type(exc).__name__}"}


def _timed(torch, fn):
    torch.cuda.synchronize()
    t = time.perf_counter()
    fn()
    torch.cuda.synchronize()
    return time.perf_counter() - t


def ceilings() -> int:
    """What a kernel that only reads memory and one that only multiplies reach on this GPU, against the published peaks."""
    import torch

    from arle_amd.kernels import ceilings as c

    read = c.read_bandwidth()
    small = c.read_bandwidth(launches=40)
    m32, m16 = c.mfma_rate(shape=32), c.mfma_rate(shape=16)
    same32 = c.mfma_rate(shape=32, random_operands=False)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    # one workgroup of four waves a busy compute unit: what a product costs in time says what the clock is (32 cycles)
    by_busy = {n: c.mfma_rate(shape=32, workgroups=n, repeats=2) for n in (cus // 8, cus // 2, 3 * cus // 4, cus)}
    print(json.dumps({
        "metric": "measured ceilings of one GPU", "unit": "GB/s and TFLOP/s",
        "hbm_read_gbs": round(read["best"] / 1e9, 1), "hbm_read_frac_of_peak": round(read["best"] / 1e9 / PEAK_HBM_GBS, 4),
        "hbm_read_100mb_launches_gbs": round(small["best"] / 1e9, 1),
        "hbm_read_by_workgroups_gbs": {str(k): round(v / 1e9, 1) for k, v in read["by_workgroups"].items()},
        "mfma_bf16_32x32x16_tflops": round(m32 / 1e12, 1), "mfma_bf16_16x16x32_tflops": round(m16 / 1e12, 1),
        "mfma_frac_of_peak": round(max(m32, m16) / PEAK_FLOPS["bf16"], 4),
        "mfma_bf16_32x32x16_same_operands_tflops": round(same32 / 1e12, 1),
        "mfma_clock_ghz_by_busy_cus": {str(n): round(v / (n * 4 * 32768.0 / 32.0) / 1e9, 2) for n, v in by_busy.items()}}))
    return 0


def mixed_8b(args) -> int:
    """Qwen3-8B shape: 32 requests decoding at 1,024 tokens of context beside one 2,048-token prompt
    that arrives in portions of 512, cut as the scheduler cuts them (aligned_portion: four steps of 32 + 512
    rows, since stopping at 480 would cost this prompt a fifth step).  Every step is launched from the last one's
    tokens on the GPU; --no-overlap: each waits for its tokens on the host.
    Reports the mean step and the tokens a second of both kinds."""
    import torch

    from arle_amd.config import Qwen3Config
    from arle_amd.engine import Engine, StepEntry
    from arle_amd.engine.scheduler import SchedulerConfig, aligned_portion
    from arle_amd.kernels import ops
    from arle_amd.sampling import Sampler, SamplingParams

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
    state = {"last": last, "chosen": None}
    sampler = Sampler(engine.device)
    greedy = [(SamplingParams(), 0, 0, [])] * (decoders + 1)
    align = 0 if args.no_overlap else SchedulerConfig().step_row_alignment
    cuts, a = [], 0
    while a < prompt:       # the portions as Scheduler.plan_prefill cuts them
        n = aligned_portion(min(prompt - a, portion), prompt - a, decoders, align)
        cuts.append((a, n))
        a += n

    def one_prompt(tag):
        engine.add_request(tag)
        toks = rand(prompt)
        for a, n in cuts:
            before = state["chosen"]
            if before is None:
                entries = [StepEntry(k, [t], [0]) for k, t in zip(keys, state["last"])]
            else:
                entries = [StepEntry(k, [before.feed(i)], [0]) for i, k in enumerate(keys)]
            last_piece = a + n == prompt
            entries.append(StepEntry(tag, toks[a:a + n], [n - 1] if last_piece else []))
            chosen = sampler.choose(engine.step(entries, borrow_logits=True), greedy[:decoders + (1 if last_piece else 0)])
            if args.no_overlap:
                state["last"] = chosen.tokens()[:decoders]
            else:
                state["chosen"] = chosen
                if before is not None:
                    state["last"] = before.tokens()[:decoders]
        engine.end_request(tag)

    def settle():
        if state["chosen"] is not None:
            state["last"], state["chosen"] = state["chosen"].tokens()[:decoders], None

    for i in range(2):          # the second pass captures the step shapes, later ones replay them
        one_prompt(("warm", i))
    settle()
    # the decoders have grown by a few tokens; the timed prompts run just above 1,024 tokens of context
    reps = max(1, args.steps // len(cuts))
    dt = _timed(torch, lambda: ([one_prompt(("p", i)) for i in range(reps)], settle()))
    steps = len(cuts) * reps
    ms = dt / steps * 1e3
    flops = sum(prefill_flops_portion(raw, a, n) for a, n in cuts) / len(cuts)
    portion = prompt / len(cuts)     # mean tokens of a portion
    line = {"metric": "mixed step: 32 decoding requests at 1,024 tokens + a 512-token prompt portion (Qwen3-8B shape)",
            "value": round(steps * (decoders + portion) / dt, 1), "unit": "tok/s", "n_gpus": 1, "steps": steps,
            "warmup": 8, "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16", "data": "synthetic: seeded random weights N(0,0.02), uniform random token ids",
            "config": {"model": "Qwen3-8B shape", "decoding_requests": decoders, "decode_context": context,
                       "prompt_len": prompt, "portions": " ".join(str(n) for _, n in cuts), "layers": raw["num_hidden_layers"],
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
    state = {"last": last, "chosen": None}
    from arle_amd.sampling import Sampler, SamplingParams
    sampler, greedy = Sampler(engine.device), [(SamplingParams(), 0, 0, [])] * batch

    def one_step():     # launched from the last step's tokens on the GPU, those read meanwhile; --no-overlap: waiting
        before = state["chosen"]
        if before is None:
            entries = [StepEntry(k, [t], [0]) for k, t in zip(keys, state["last"])]
        else:
            entries = [StepEntry(k, [before.feed(i)], [0]) for i, k in enumerate(keys)]
        chosen = sampler.choose(engine.step(entries, borrow_logits=True), greedy)
        if args.no_overlap:
            state["last"] = chosen.tokens()
        else:
            state["chosen"] = chosen
            if before is not None:
                state["last"] = before.tokens()

    def settle():
        if state["chosen"] is not None:
            state["last"], state["chosen"] = state["chosen"].tokens(), None

    for _ in range(warmup):
        one_step()
    settle()
    ctx0 = engine.length(keys[0])
    dt = _timed(torch, lambda: ([one_step() for _ in range(steps)], settle()))
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


def step_gaps(args) -> int:
    """Decode steps of the Qwen3-4B shape both ways, steps that wait for their tokens on the host and steps launched
    from the last one's tokens on the GPU: milliseconds a step, and from a kernel timeline of six steps how long
    the GPU works and how long it idles between kernels in a step.  One JSON line a batch size."""
    import torch
    from torch.profiler import ProfilerActivity, profile

    from arle_amd.config import Qwen3Config
    from arle_amd.engine import Engine, StepEntry
    from arle_amd.kernels import ops
    from arle_amd.sampling import Sampler, SamplingParams

    raw = dict(QWEN3_4B, num_hidden_layers=args.layers)
    config = Qwen3Config.from_dict(raw)
    batches = [args.batch] if args.batch else [1, 8, 64]
    most = max(batches)
    engine = Engine.from_config("Qwen3ForCausalLM", config, seed=0, std=0.02, dtype="bfloat16", page_size=PAGE,
                                max_tokens=most * (PROMPT + 256), max_slots=most, max_request_tokens=PROMPT + 256)
    sampler = Sampler(engine.device)
    gen = torch.Generator().manual_seed(1234)
    for batch in batches:
        keys, last = [("g", batch, i) for i in range(batch)], []
        rows = [(SamplingParams(), 0, 0, [])] * batch
        for k in keys:
            engine.add_request(k)
            toks = torch.randint(0, config.vocab_size, (PROMPT,), generator=gen).tolist()
            last.append(int(ops.argmax_rows(engine.step([StepEntry(k, toks, [PROMPT - 1])]))[0]))
        state = {"last": last, "chosen": None}

        def waiting():
            out = engine.step([StepEntry(k, [t], [0]) for k, t in zip(keys, state["last"])])
            state["last"] = sampler.choose(out, rows).tokens()

        def ahead():
            before = state["chosen"]
            if before is None:
                entries = [StepEntry(k, [t], [0]) for k, t in zip(keys, state["last"])]
            else:
                entries = [StepEntry(k, [before.feed(i)], [0]) for i, k in enumerate(keys)]
            state["chosen"] = sampler.choose(engine.step(entries, borrow_logits=True), rows)
            if before is not None:
                state["last"] = before.tokens()

        def settle():
            if state["chosen"] is not None:
                state["last"], state["chosen"] = state["chosen"].tokens(), None

        line = {"metric": f"decode step at batch {batch}, {PROMPT}-token prompts (Qwen3-4B shape): steps that wait "
                          f"for their tokens and steps launched ahead", "unit": "ms a step", "n_gpus": 1, "dtype": "bf16",
                "layers": args.layers}
        for name, fn in (("waiting", waiting), ("ahead", ahead)):
            for _ in range(8):
                fn()
            settle()
            wall = _timed(torch, lambda: ([fn() for _ in range(args.steps)], settle())) / args.steps
            with profile(activities=[ProfilerActivity.CUDA]) as prof:
                for _ in range(7):
                    fn()
                settle()
                torch.cuda.synchronize()
            evs = sorted((e for e in prof.events() if e.device_type == torch.autograd.DeviceType.CUDA),
                         key=lambda e: e.time_range.start)
            first = [i for i, e in enumerate(evs) if "embed_gather" in e.name]
            evs = evs[first[1]:first[-1]]          # whole steps 2..6: the first carries the profiler's start
            n = len(first) - 2
            busy = sum(e.time_range.end - e.time_range.start for e in evs) / n
            span = (evs[-1].time_range.end - evs[0].time_range.start) / n
            line[name] = {"ms_per_step": round(wall * 1e3, 4), "gpu_busy_us": round(busy, 1), "gpu_idle_us": round(span - busy, 1),
                          "kernels": round(len(evs) / n, 1)}
        print(json.dumps(line), flush=True)
        for k in keys:
            engine.end_request(k)
    return 0


def first_token(args) -> int:
    """Time to the first token through `LLM.generate` (scheduler, sampler, engine) for one prompt of 2,048, 8,192 and
    16,000 tokens and for four prompts of 2,048 at once, with the portion size that the GPU's memory gives (the
    default) and with portions of 512: one JSON line each."""
    import torch

    from arle_amd.config import Qwen3Config
    from arle_amd.engine import Engine
    from arle_amd.engine.api import LLM

    raw = dict(QWEN3_4B, num_hidden_layers=args.layers)
    config = Qwen3Config.from_dict(raw)
    longest = 16384 + 64
    engine = Engine.from_config("Qwen3ForCausalLM", config, seed=0, std=0.02, dtype="bfloat16", page_size=PAGE,
                                max_tokens=4 * longest, max_slots=4, max_request_tokens=longest)
    gen = torch.Generator().manual_seed(1234)
    rand = lambda n: torch.randint(0, config.vocab_size, (n,), generator=gen).tolist()
    for chunk in (None, 512):
        llm = LLM(engine, num_slots=4, chunked_prefill_size=chunk, max_seq_len=longest)
        for prompts in ([2048], [8192], [16000], [2048] * 4):
            batch = [rand(n) for n in prompts]
            for _ in range(3):      # the third run replays what the first two captured
                outs = llm.generate(batch, max_tokens=4, ignore_eos=True)
            ttft = max(o.ttft_s for o in outs)
            print(json.dumps({"metric": f"time to the first token of {len(prompts)} prompt(s) of {prompts[0]:,} tokens "
                                        f"through LLM.generate (Qwen3-4B shape)", "value": round(ttft * 1e3, 2), "unit": "ms",
                              "higher_is_better": False, "n_gpus": 1, "dtype": "bf16", "layers": args.layers,
                              "chunked_prefill_size": llm.sched_config.chunked_prefill_size,
                              "prefill_steps": llm.last_stats["steps"]["prefill"],
                              "prompt_tok_s": round(sum(prompts) / ttft, 1)}), flush=True)
    return 0


def generate_workload(args) -> int:
    """The decode workload of the baseline's benchmark configuration as a user runs it: 1, 8 and 64 prompts of 2,048
    uniform-random tokens, 256 tokens generated for each, through `LLM.generate` (scheduler, sampler, engine; greedy
    and at temperature 0.8).  One JSON line each: generated tokens a second after the first token, the time to the
    first token of the last prompt served, and the steps by kind."""
    import torch

    from arle_amd.config import Qwen3Config
    from arle_amd.engine import Engine
    from arle_amd.engine.api import LLM

    config = Qwen3Config.from_dict(dict(QWEN3_4B, num_hidden_layers=args.layers))
    prompt, new, most = args.prompt_len, 256, 64
    longest = -(-(prompt + new + 1) // 64) * 64
    engine = Engine.from_config("Qwen3ForCausalLM", config, seed=0, std=0.02, dtype="bfloat16", page_size=args.page_size,
                                max_tokens=most * longest, max_slots=most, max_request_tokens=longest)
    gen = torch.Generator().manual_seed(1234)
    for temperature in (0.0, 0.8):
        for n in (1, 8, most):
            llm = LLM(engine, num_slots=most, max_seq_len=longest)
            prompts = [torch.randint(0, config.vocab_size, (prompt,), generator=gen).tolist() for _ in range(n)]
            for _ in range(3):      # the third run replays what the first two captured (a shape is captured when it repeats)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                outs = llm.generate(prompts, max_tokens=new, temperature=temperature, seed=3, ignore_eos=True)
                torch.cuda.synchronize()
                wall = time.perf_counter() - t0
            ttft = max(o.ttft_s for o in outs)
            made = sum(o.usage.completion_tokens for o in outs)
            print(json.dumps({"metric": f"{n} prompt(s) of {prompt:,} tokens, {new} generated each, through LLM.generate "
                                        f"(Qwen3-4B shape, temperature {temperature})",
                              "value": round((made - n) / (wall - ttft), 1), "unit": "generated tok/s after the first token",
                              "higher_is_better": True, "n_gpus": 1, "dtype": "bf16", "layers": args.layers,
                              "wall_s": round(wall, 4), "ttft_ms": round(ttft * 1e3, 1),
                              "ms_per_token_a_request": round(sum(o.tpot_s for o in outs) / n * 1e3, 3),
                              "steps": llm.last_stats["steps"]}), flush=True)
    return 0


def tune_products(args) -> int:
    """Measure the table of `arle_amd.kernels.tune` for one model's widths and write it; one line a (product, row
    count) to stderr, and at the end what the table gains over the rules at every row count where they differ."""
    from arle_amd.kernels import tune

    named = {"4b": (2560, 4096, 1024, 9728, 151936), "8b": (4096, 4096, 1024, 12288, 151936),
             "32b": (5120, 8192, 1024, 25600, 151936)}
    widths = named.get(args.tune_products) or tuple(int(v) for v in args.tune_products.split(","))
    if len(widths) not in (4, 5):
        print("--tune-products takes 4b, 8b, 32b or hidden,q_width,kv_width,intermediate[,vocabulary]", file=sys.stderr)
        return 2

    def say(rec):
        print(f"[tune] {rec['product']:8s} rows {rec['rows']:5d}: rule {rec['rule'][0]:13s} {rec['rule_us']:8.1f} us   "
              f"best {rec['best'][0]:13s} {rec['best_us']:8.1f} us", file=sys.stderr, flush=True)

    table, report = tune.tune_products(tune.model_products(*widths), tiled=not args.no_weight_tiles, say=say)
    path = args.out or f"product_table_{args.tune_products.replace(',', '_')}.json"
    if os.path.exists(path):       # a file may hold the tables of several runs (with and without operand tiles)
        with open(path, encoding="utf-8") as fh:
            table = {**json.load(fh), **table}
    tune.write_table(path, table)
    changed = [r for r in report if r["best"] != r["rule"]]
    print(json.dumps({"table": path, "points": len(report), "points_where_the_table_differs": len(changed),
                      "gain_us": {f"{r['product']}@{r['rows']}": round(r["rule_us"] - r["best_us"], 1) for r in changed}}))
    return 0


def sweep(args) -> int:
    """Further sizes of the Qwen3-4B shape, one JSON line each with its fraction of the roofline: decode at batch 16
    and 32 (2,048-token prompts), at batch 128 and 256 (1,024 tokens of context), at batch 8 with 8,192, 16,384 and
    32,768 tokens of context, at batch 64 with 16,384, prefills of 32,768, 16,384, 8,192, 512 and 128 tokens, and a
    504-token prompt portion beside 8 decoding requests."""
    import torch

    from arle_amd.config import Qwen3Config
    from arle_amd.engine import Engine, StepEntry
    from arle_amd.kernels import ops

    raw = dict(QWEN3_4B, num_hidden_layers=args.layers)
    config = Qwen3Config.from_dict(raw)
    longest = 32768 + args.steps + 16     # the longest context, its warm-up and timed steps
    most_tokens = max(8 * longest + 40 * 4096, 64 * (16384 + args.steps + 16), 256 * (1024 + args.steps + 16))
    engine = Engine.from_config("Qwen3ForCausalLM", config, seed=0, std=0.02, dtype="bfloat16", page_size=PAGE,
                                max_tokens=most_tokens, max_slots=257, max_request_tokens=longest)
    gen = torch.Generator().manual_seed(1234)
    rand = lambda n: torch.randint(0, config.vocab_size, (n,), generator=gen).tolist()
    from arle_amd.sampling import Sampler, SamplingParams
    sampler, greedy_rows = Sampler(engine.device), [(SamplingParams(), 0, 0, [])] * 257
    base = {"n_gpus": 1, "dtype": "bf16", "higher_is_better": True, "data": "synthetic", "layers": args.layers}

    def fill(keys, context, portion=8192):
        last = []
        for k in keys:
            engine.add_request(k)
            toks = rand(context)
            for a in range(0, context, portion):
                piece = toks[a:a + portion]
                out = engine.step([StepEntry(k, piece, [len(piece) - 1] if a + portion >= context else [])])
            last.append(int(ops.argmax_rows(out)[0]))
        return last

    def decode_point(batch, context, steps):
        keys = [("s", batch, context, i) for i in range(batch)]
        state = {"last": fill(keys, context)}

        def one_step():     # as the headline run: launched from the last step's tokens on the GPU, those read meanwhile
            before = state.get("chosen")
            if before is None:
                entries = [StepEntry(k, [t], [0]) for k, t in zip(keys, state["last"])]
            else:
                entries = [StepEntry(k, [before.feed(i)], [0]) for i, k in enumerate(keys)]
            state["chosen"] = sampler.choose(engine.step(entries, borrow_logits=True), greedy_rows[:batch])
            if before is not None:
                state["last"] = before.tokens()

        def settle():
            state["last"] = state.pop("chosen").tokens()

        for _ in range(6):
            one_step()
        settle()
        dt = _timed(torch, lambda: ([one_step() for _ in range(steps)], settle())) / steps
        ctx = engine.length(keys[0]) - steps / 2.0
        for k in keys:
            engine.end_request(k)
        got = decode_bytes(raw, batch, ctx) / dt / 1e9
        print(json.dumps(dict(base, metric=f"decode tok/s at batch {batch}, {context}-token context (Qwen3-4B shape)",
                              value=round(batch / dt, 1), unit="tok/s", ms_per_step=round(dt * 1e3, 4), steps=steps,
                              roofline={"bound": "hbm", "achieved": round(got, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                        "frac": round(got / PEAK_HBM_GBS, 4)})), flush=True)

    def prefill_point(tokens):
        def once(tag):
            engine.add_request(tag)
            toks = rand(tokens)
            dt = _timed(torch, lambda: ops.argmax_rows(engine.step([StepEntry(tag, toks, [tokens - 1])])))
            engine.end_request(tag)
            return dt

        once(("w", tokens, 0)), once(("w", tokens, 1))
        dt = min(once(("p", tokens, i)) for i in range(3))
        print(json.dumps(dict(base, metric=f"prefill tok/s at {tokens} tokens (Qwen3-4B shape)", value=round(tokens / dt, 1),
                              unit="tok/s", ms=round(dt * 1e3, 3),
                              frac=round(prefill_flops(raw, tokens) / dt / PEAK_FLOPS["bf16"], 4))), flush=True)

    def mixed_point(decoders, context, portion, prompt):
        keys = [("m", i) for i in range(decoders)]
        state = {"last": fill(keys, context)}

        def one_prompt(tag):
            engine.add_request(tag)
            toks = rand(prompt)
            for a in range(0, prompt, portion):
                entries = [StepEntry(k, [t], [0]) for k, t in zip(keys, state["last"])]
                entries.append(StepEntry(tag, toks[a:a + portion], [portion - 1] if a + portion == prompt else []))
                state["last"] = ops.argmax_rows(engine.step(entries)).tolist()[:decoders]
            engine.end_request(tag)

        one_prompt(("mw", 0)), one_prompt(("mw", 1))
        reps, per = 4, prompt // portion
        dt = _timed(torch, lambda: [one_prompt(("mp", i)) for i in range(reps)]) / (reps * per)
        for k in keys:
            engine.end_request(k)
        flops = 2.0 * (decoders + portion) * (raw["num_hidden_layers"] * layer_params(raw) ) + 2.0 * raw["vocab_size"] * raw["hidden_size"] * (decoders + 1)
        print(json.dumps(dict(base, metric=f"mixed step: {decoders} decoding requests at {context} tokens + a {portion}-token "
                                           f"prompt portion (Qwen3-4B shape)", value=round((decoders + portion) / dt, 1),
                              unit="tok/s", ms_per_step=round(dt * 1e3, 4), decode_tok_s=round(decoders / dt, 1),
                              prefill_tok_s=round(portion / dt, 1), frac_of_matrix_peak=round(flops / dt / PEAK_FLOPS["bf16"], 4),
                              frac_of_hbm_peak=round(decode_bytes(raw, decoders, context + 64) / dt / 1e9 / PEAK_HBM_GBS, 4))),
              flush=True)

    for batch in (16, 32):
        decode_point(batch, 2048, args.steps)
    decode_point(128, 1024, args.steps)
    decode_point(256, 1024, args.steps)
    for context in (8192, 16384, 32768):
        decode_point(8, context, args.steps)
    decode_point(64, 16384, min(args.steps, 16))
    prefill_point(32768)
    prefill_point(16384)
    prefill_point(8192)
    prefill_point(512)
    prefill_point(128)
    mixed_point(8, 2048, 504, 2016)      # the first four portions of a long prompt as the scheduler cuts it beside 8 decoding requests: 512 rows a step
    return 0


def main() -> int:
    global PAGE, PROMPT
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
    ap.add_argument("--no-overlap", action="store_true",
                    help="decode steps wait for their tokens on the host before the next is prepared (default: the "
                         "next step is launched from the tokens on the GPU, as the scheduler does)")
    ap.add_argument("--no-weight-tiles", action="store_true",
                    help="without the second copy of the projection weights that the few-rows kernels stream")
    ap.add_argument("--no-parts", action="store_true",
                    help="skip the breakdown of the step's time by part of the model (a profiled step)")
    ap.add_argument("--parts-only", action="store_true",
                    help="print only that breakdown (what the default run starts as a child process, after its own timing)")
    ap.add_argument("--ceilings", action="store_true",
                    help="measure what a kernel that only reads, and one that only multiplies, reach on this GPU, and exit")
    ap.add_argument("--prompt-len", type=int, default=PROMPT,
                    help="tokens of the prefill that --prefill-only measures and of the prompts of --generate (default 2,048)")
    ap.add_argument("--prefill-only", action="store_true",
                    help="measure the 2,048-token prefill alone (for profiles of its kernels) and print that")
    ap.add_argument("--gaps", action="store_true",
                    help="decode steps that wait for their tokens against steps launched ahead: time a step, GPU busy and idle")
    ap.add_argument("--first-token", action="store_true",
                    help="time to the first token through LLM.generate, portions by the GPU's memory against portions of 512")
    ap.add_argument("--generate", action="store_true",
                    help="the decode workload as a user runs it: 1, 8 and 64 prompts of --prompt-len tokens, 256 generated each, "
                         "through LLM.generate")
    ap.add_argument("--sweep", action="store_true",
                    help="further sizes of the Qwen3-4B shape (batch 16/32, 8k/32k context, 8,192-token prefill, portions "
                         "beside decoding requests), one JSON line each")
    ap.add_argument("--tune-products", metavar="WIDTHS", default=None,
                    help="time every kernel that can run each of a layer's four matrix products, row count by row count, "
                         "and write the table that ARLE_AMD_PRODUCT_TABLE / ops.load_product_table reads; WIDTHS: 4b, 8b, "
                         "32b or hidden,q_width,kv_width,intermediate[,vocabulary]")
    ap.add_argument("--out", default=None, help="--tune-products: the table's file (default: product_table_<widths>.json)")
    ap.add_argument("--workload", default="qwen3-4b", choices=["qwen3-4b", "qwen3-8b-mixed", "qwen3-32b-decode"],
                    help="qwen3-4b is the default run; the other two are further workloads at larger shapes")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this engine has no multi-GPU path (asked for --gpus {args.gpus})")
        return 2
    PAGE = args.page_size
    if args.prefill_only:
        PROMPT = args.prompt_len
    if args.ceilings:
        return ceilings()
    if args.tune_products:
        return tune_products(args)
    if args.sweep:
        return sweep(args)
    if args.first_token:
        return first_token(args)
    if args.generate:
        return generate_workload(args)
    if args.gaps:
        return step_gaps(args)
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
    from arle_amd.sampling import Sampler, SamplingParams

    raw = dict(QWEN3_4B, num_hidden_layers=args.layers)
    config = Qwen3Config.from_dict(raw)
    dkey = "bf16" if args.dtype == "bfloat16" else "fp32"
    elt = 2 if dkey == "bf16" else 4
    max_batch = args.batch if (args.no_points or args.parts_only or args.prefill_only) else max(args.batch, 64)
    longest = max(CONTEXT, PROMPT + 64)    # --prompt-len may ask for a longer prefill than the default run's context
    t0 = time.time()
    engine = Engine.from_config("Qwen3ForCausalLM", config, seed=0, std=0.02, dtype=args.dtype,
                                page_size=PAGE, max_tokens=(max_batch + 1) * longest, max_slots=max_batch + 1,
                                max_request_tokens=longest, weight_tiles=False if args.no_weight_tiles else None)
    print(f"[bench] engine ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    gen = torch.Generator().manual_seed(1234)
    sampler = Sampler(engine.device)       # the product's sampler: greedy rows are one argmax kernel, read back on its own stream
    greedy_rows = [(SamplingParams(), 0, 0, [])] * (max_batch + 1)

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


    for i in range(5):      # eager, captured, then replays until the clocks have settled (the sixth run is as fast as the twentieth)
        prefill_once(("warm", i))
    prefill_s = min(prefill_once(("prefill", i)) for i in range(5))
    prefill = {"value": round(PROMPT / prefill_s, 1), "tokens": PROMPT, "ms": round(prefill_s * 1e3, 3),
               "frac": round(prefill_flops(raw, PROMPT) / prefill_s / PEAK_FLOPS[dkey], 4)}
    print(f"[bench] prefill {prefill}", file=sys.stderr, flush=True)
    if args.prefill_only:
        print(json.dumps({"metric": f"prefill tok/s at {PROMPT} tokens (Qwen3-4B shape, random weights)",
                          "value": prefill["value"], "unit": "tok/s", "n_gpus": 1, "dtype": dkey,
                          "higher_is_better": True, "prefill": prefill}))
        return 0

    # ---- decode ---------------------------------------------------------------------------------
    def decode_run(batch, steps, warmup, parts=False):
        """(seconds of `steps` timed steps, mean context); with `parts` instead the breakdown of a step's time."""
        keys = [("d", batch, i) for i in range(batch)]
        last = []
        for k in keys:
            engine.add_request(k)
        per_step = max(1, 8192 // PROMPT)
        for i in range(0, batch, per_step):   # real prefill of every request, a few prompts a step
            group = keys[i:i + per_step]
            out = engine.step([StepEntry(k, prompt_tokens(PROMPT), [PROMPT - 1]) for k in group])
            last.extend(ops.argmax_rows(out).tolist())
        state = {"last": last, "chosen": None}

        def one_step():
            """A decode step as the scheduler runs it (Scheduler._run_ahead): launched from the tokens that the
            step before left on the GPU, which the host reads back while this step runs.  --no-overlap: every
            step waits for its tokens on the host before the next is prepared."""
            if args.no_overlap or parts:
                out = engine.step([StepEntry(k, [t], [0]) for k, t in zip(keys, state["last"])])
                state["last"] = ops.argmax_rows(out).tolist()   # the host needs the token to go on
                return
            before = state["chosen"]
            if before is None:
                entries = [StepEntry(k, [t], [0]) for k, t in zip(keys, state["last"])]
            else:
                entries = [StepEntry(k, [before.feed(i)], [0]) for i, k in enumerate(keys)]
            state["chosen"] = sampler.choose(engine.step(entries, borrow_logits=True), greedy_rows[:batch])
            if before is not None:
                state["last"] = before.tokens()                 # the step before: every token reaches the host

        def settle():
            if state["chosen"] is not None:
                state["last"] = state["chosen"].tokens()
                state["chosen"] = None

        for _ in range(warmup):
            one_step()
        ctx0 = engine.length(keys[0])
        settle()
        dt = timed(lambda: ([one_step() for _ in range(steps)], settle()))   # the last step's tokens are read inside
        ctx_mean = ctx0 + (steps - 1) / 2.0 + 1
        if parts:
            from arle_amd.kernels import ceilings as measured

            read_ceiling = measured.read_bandwidth(total_bytes=1 << 30, repeats=3)["best"]
            mfma_ceiling = max(measured.mfma_rate(shape=32, iters=4000, repeats=2),
                               measured.mfma_rate(shape=16, iters=4000, repeats=2))
            ctx_now = engine.length(keys[0]) + 2
            calls = [lambda: prefill_once(("parts", 0))] * 3 + [one_step] * 5
            traced = profiled_steps(torch, calls)
            out = {"ceilings": {"hbm_read_gbs": round(read_ceiling / 1e9, 1), "mfma_tflops": round(mfma_ceiling / 1e12, 1)}}
            times = part_times(traced[:3], args.layers)
            flops = part_flops_prefill(raw, PROMPT)
            head_flops = flops.pop("head")      # one row against the whole table: a stream of weights, judged by its bytes
            us, of_peak, of_ceiling = part_report(times, flops, PEAK_FLOPS[dkey], mfma_ceiling)
            head_bytes = raw["vocab_size"] * raw["hidden_size"] * elt
            of_peak["head_hbm"] = round(head_bytes / (times["head"] * 1e-6) / (PEAK_HBM_GBS * 1e9), 4)
            of_ceiling["head_hbm"] = round(head_bytes / (times["head"] * 1e-6) / read_ceiling, 4)
            # the profiled pass is longer than the timed one (the profiler's own cost a kernel): both are given
            us["sum"] = round(sum(v for k, v in us.items() if k != "kernels"), 1)
            out.update(prefill_parts_us=us, prefill_parts_frac_peak=of_peak, prefill_parts_frac_ceiling=of_ceiling)
            us, of_peak, of_ceiling = part_report(part_times(traced[3:], args.layers),
                                                  part_bytes_decode(raw, batch, ctx_now, elt), PEAK_HBM_GBS * 1e9, read_ceiling)
            us["sum"] = round(sum(v for k, v in us.items() if k != "kernels"), 1)
            out.update(decode_parts_us=us, decode_parts_frac_peak=of_peak, decode_parts_frac_ceiling=of_ceiling)
            for k in keys:
                engine.end_request(k)
            return out
        for k in keys:
            engine.end_request(k)
        return dt, ctx_mean

    if args.parts_only:
        print(json.dumps(decode_run(args.batch, 4, 6, parts=True)))
        return 0
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
                   "page_size": PAGE, "weight_tiles": engine.rt.weight_tiles,
                   "readback_lag_steps": 0 if args.no_overlap else 1},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4)},
        "points": points,
    }
    if not args.no_parts and dkey == "bf16":
        line.update(parts_in_a_child_process(args))
        # the parts come from a second, profiled run: their sums stand beside the timed steps they are read against
        if isinstance(line.get("prefill_parts_us"), dict):
            line["prefill_parts_us"]["timed_step"] = round(prefill["ms"] * 1e3, 1)
            line["decode_parts_us"]["timed_step"] = round(ms_per_step * 1e3, 1)
    if args.batch != 8:
        line["metric"] = line["metric"].replace("batch 8", f"batch {args.batch}")
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
