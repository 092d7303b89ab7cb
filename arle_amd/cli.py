"""Command line in the manner of the reference's `arle`:

    arle-amd --model-path DIR [--max-tokens N] [--temperature T] run (--prompt S | --stdin | --prompt-ids 1,2,3) [--json]

Global options and `run` follow crates/cli/src/args.rs:188-302: `--model-path`, `--max-tokens`
(0 or `auto`: the model's max_position_embeddings, crates/cli/src/lib.rs:240-266), `--temperature`
(default 0.0 = greedy); `run --prompt/--stdin/--json`.  The engine options carry the names of the
`infer` binary's flags (infer/src/main.rs:26-236): `--num-slots`, `--max-seq-len`,
`--chunked-prefill-size`, `--max-num-batched-tokens`, `--max-prefill-tokens`, `--prefill-max-requests`,
`--mem-fraction-static`.
After the answer, one summary line goes to stderr: prompt tok/s (= prompt tokens / TTFT), TTFT and
output tok/s (crates/cli/src/tps.rs:1-60).  `--prompt-ids` is this engine's own: folders written by
the random-weights mode have no tokenizer.
"""
from __future__ import annotations

import argparse
import json
import sys
import time


def _max_tokens(value: str) -> int:
    if value.strip().lower() == "auto":
        return 0
    n = int(value)
    if n < 0:
        raise argparse.ArgumentTypeError("--max-tokens must be >= 0 (0 = auto)")
    return n


def _num_slots(value: str):
    if value.strip().lower() == "auto":
        return None
    n = int(value)
    if n < 1:
        raise argparse.ArgumentTypeError("--num-slots must be at least 1 (or auto)")
    return n


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="arle-amd", description="Qwen3 inference on one MI355X")
    ap.add_argument("--model-path", required=False, help="model folder (config.json + safetensors)")
    ap.add_argument("--max-tokens", type=_max_tokens, default=0,
                    help="tokens to generate; 0/auto = the model's max_position_embeddings")
    ap.add_argument("--temperature", type=float, default=0.0, help="sampling temperature (0.0 = greedy)")
    ap.add_argument("--top-k", type=int, default=-1)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--min-p", type=float, default=0.0)
    ap.add_argument("--seed", type=int, default=42)
    ap.add_argument("--ignore-eos", action="store_true")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--num-slots", type=_num_slots, default=4,
                    help="requests that run at a time; auto: as many of --max-seq-len as the cache holds, 4 to 128")
    ap.add_argument("--max-seq-len", type=int, default=None)
    ap.add_argument("--chunked-prefill-size", type=int, default=None,
                    help="longest prompt portion of one request in a step; default: by the GPU's memory "
                         "(<35 GiB 2048, <60 4096, <90 8192, else 16384)")
    ap.add_argument("--max-num-batched-tokens", type=int, default=16384)
    ap.add_argument("--max-prefill-tokens", type=int, default=None,
                    help="prompt tokens of all requests in a step; default: --max-num-batched-tokens")
    ap.add_argument("--prefill-max-requests", type=int, default=None)
    ap.add_argument("--kv-cache-tokens", type=int, default=None,
                    help="tokens the paged cache holds (default: sized from free GPU memory, see --mem-fraction-static)")
    ap.add_argument("--mem-fraction-static", type=float, default=0.85,
                    help="share of the GPU's memory that weights and cache may take together; the rest is headroom")
    ap.add_argument("--page-size", type=int, default=None)
    ap.add_argument("--no-cuda-graph", action="store_true",
                    help="launch every step kernel by kernel instead of replaying captured HIP graphs")
    ap.add_argument("--warm-up", action="store_true",
                    help="capture the decode graphs of every batch size before the first request (the reference's "
                         "server does so when it starts; a single prompt gains nothing from it)")
    ap.add_argument("--tune-products", metavar="FILE", default=None,
                    help="measure which kernel runs each matrix product of this model fastest, go by that and write the "
                         "table to FILE (read again with ARLE_AMD_PRODUCT_TABLE=FILE); about a minute")
    ap.add_argument("--no-weight-tiles", action="store_true",
                    help="do not keep the second, decode-friendly copy of the projection weights")
    sub = ap.add_subparsers(dest="command")
    run = sub.add_parser("run", help="run a single prompt and exit")
    src = run.add_mutually_exclusive_group()
    src.add_argument("--prompt", help="prompt text (needs tokenizer.json in the model folder)")
    src.add_argument("--stdin", action="store_true", help="read the prompt text from stdin")
    src.add_argument("--prompt-ids", help="prompt as comma-separated token ids")
    run.add_argument("--json", action="store_true", help="print one JSON document")
    init = sub.add_parser("random-weights", help="write a model folder with seeded random weights")
    init.add_argument("--config", required=True, help="a config.json to take the sizes from")
    init.add_argument("--out", required=True)
    init.add_argument("--seed-weights", type=int, default=0)
    init.add_argument("--std", type=float, default=0.02)
    init.add_argument("--norm-std", type=float, default=0.0)
    return ap


def _run(argv=None) -> int:
    args = build_parser().parse_args(argv)
    if args.command == "random-weights":
        from . import models  # noqa: F401
        from .config.base import read_json_file
        from .config.registry import detect_architecture
        from .weights import write_random_model

        raw = read_json_file(args.config)
        arch = detect_architecture(raw)
        write_random_model(args.out, arch.name, arch.config_class.from_dict(raw), args.seed_weights,
                           args.std, args.norm_std)
        print(args.out)
        return 0
    if args.command != "run":
        build_parser().print_help()
        return 2
    if not args.model_path:
        print("error: --model-path is required", file=sys.stderr)
        return 2

    from .engine.api import LLM
    from .sampling import SamplingParams

    llm = LLM(args.model_path, dtype=args.dtype, num_slots=args.num_slots, max_seq_len=args.max_seq_len,
              chunked_prefill_size=args.chunked_prefill_size,
              max_num_batched_tokens=args.max_num_batched_tokens, max_prefill_tokens=args.max_prefill_tokens,
              prefill_max_requests=args.prefill_max_requests, kv_cache_tokens=args.kv_cache_tokens,
              page_size=args.page_size, seed=args.seed, cuda_graph=not args.no_cuda_graph,
              mem_fraction_static=args.mem_fraction_static,
              weight_tiles=False if args.no_weight_tiles else None, warm_up=args.warm_up,
              tune_products=args.tune_products or False)
    if args.prompt_ids:
        prompt = [int(t) for t in args.prompt_ids.replace(" ", "").split(",") if t]
    else:
        prompt = sys.stdin.read() if args.stdin else args.prompt
        if prompt is None:
            print("error: give --prompt, --stdin or --prompt-ids", file=sys.stderr)
            return 2
    max_tokens = args.max_tokens or llm.engine.spec.max_positions
    params = SamplingParams(temperature=args.temperature, top_k=args.top_k, top_p=args.top_p,
                            min_p=args.min_p, ignore_eos=args.ignore_eos)
    t0 = time.perf_counter()
    if args.json or llm.tokenizer is None:
        out = llm.generate([prompt], max_tokens=max_tokens, sampling=params)[0]
    else:       # text goes out as it is generated, as the reference's prompt loop prints it (crates/cli/src/repl.rs:760-800)
        first = None

        def shown(deltas):
            nonlocal first
            for d in deltas:
                if first is None and d.token_ids:
                    first = time.perf_counter() - t0
                if d.text_delta:
                    sys.stdout.write(d.text_delta)
                    sys.stdout.flush()
                yield d

        out = llm._collect([prompt], shown(llm.generate_stream([prompt], max_tokens=max_tokens, sampling=params)))[0]
        out.ttft_s = first
        print()
    elapsed = time.perf_counter() - t0
    if args.json:
        print(json.dumps({"model": args.model_path, "backend": "hip-gfx950", "text": out.text,
                          "token_ids": out.response_token_ids, "finish_reason": out.finish_reason,
                          "usage": {"prompt_tokens": out.usage.prompt_tokens,
                                    "completion_tokens": out.usage.completion_tokens,
                                    "total_tokens": out.usage.total_tokens}}))
    elif llm.tokenizer is None:
        print(" ".join(str(t) for t in out.response_token_ids))
    ttft = out.ttft_s or elapsed
    decode_time = max(elapsed - ttft, 1e-9)
    print(f"prompt {out.usage.prompt_tokens / max(ttft, 1e-9):.1f} tok/s | TTFT {ttft * 1e3:.1f} ms | "
          f"output {max(out.usage.completion_tokens - 1, 0) / decode_time:.1f} tok/s "
          f"({out.usage.completion_tokens} tokens, {out.finish_reason})", file=sys.stderr)
    return 0


def main(argv=None) -> int:
    """The command line; what the user can mend (a folder that is not a model, a damaged file, a prompt that does
    not fit, a missing compiler) ends in one line `error: ...` and exit code 1, not in a traceback."""
    from .cache.manager import NoFreeSlot
    from .cache.pages import OutOfPages
    from .engine.engine import EngineError
    from .kernels.build import BuildError

    try:
        return _run(argv)
    except (ValueError, OSError, EngineError, OutOfPages, NoFreeSlot, BuildError) as exc:
        print(f"error: {exc}", file=sys.stderr)
        return 1


if __name__ == "__main__":
    sys.exit(main())
