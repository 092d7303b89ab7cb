"""The engine: a model, its cache, and the one step function everything else is built on.

`step(entries)` takes a batch of (request, its next tokens, wanted places): portions of
prompts beside single decoded tokens, cut anywhere.  It makes room in the cache for all of
them or for none, runs only the rows it is given against the cache earlier steps left,
and returns float32 logits at the wanted places, in the order of the entries and of their
`want` lists.  The reference splits this over three calls (prefill batch, decode batch,
mixed batch: infer/src/model/qwen3/forward.rs:376-400,605-637,650-665); here a decoded token
is an entry of one token and there is one call.
"""
from __future__ import annotations

import os

import torch

from .. import models  # noqa: F401  (registers the architectures)
from ..cache.manager import (CacheManager, OutOfPages, PagedNeed, cache_bytes_per_token, pages_for_memory, slots_for_tokens,
                             state_bytes_per_slot)
from ..config.registry import detect_architecture, load_model_config
from ..models.decoder import DEBUG_DUMP_ENV, build_model, expected_checkpoint_tensors
from ..parts.base import Runtime
from ..weights.loader import load_weights
from ..weights.random_init import random_weights
from ..kernels import ops
from .batch import DeviceToken, StepEntry, build_step_batch, packed_size

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32,
          "fp32": torch.float32}
DEFAULT_PAGE_SIZE = 16  # tokens per page, as the reference's bf16 pool (crates/cuda-kernels/src/kv_types.rs:53-59)
DEFAULT_MEM_FRACTION_STATIC = 0.85   # infer/src/scheduler/types.rs:215


class EngineError(RuntimeError):
    pass


def decode_warmup_sizes(max_batch: int) -> list:
    """The batch sizes whose decode graphs are captured ahead: every size up to 64, then every sixteenth from 80 on,
    and the largest itself (infer/src/scheduler/cuda/core/warmup.rs:267-285)."""
    sizes = list(range(1, min(64, max_batch) + 1))
    sizes += list(range(80, max_batch + 1, 16))
    if sizes and sizes[-1] != max_batch and max_batch > 8:
        sizes.append(max_batch)
    return sizes


def _device(device=None) -> torch.device:
    if not torch.cuda.is_available():
        raise EngineError("arle_amd needs a GPU: torch.cuda.is_available() is False and there is "
                          "no CPU path")
    return torch.device(device or "cuda:0")


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        return name
    try:
        return DTYPES[str(name)]
    except KeyError:
        raise EngineError(f"unknown dtype {name!r}; use bfloat16 or float32") from None


class Engine:
    def __init__(self, spec, tensors: dict, *, dtype=torch.bfloat16, device=None,
                 page_size: int = DEFAULT_PAGE_SIZE, max_tokens: int | None = None,
                 num_pages: int | None = None, max_slots: int | None = 4,
                 max_request_tokens: int | None = None, cuda_graph: bool = True,
                 weight_tiles: bool | None = None, mem_fraction_static: float = DEFAULT_MEM_FRACTION_STATIC,
                 product_table=None):
        """
        max_tokens: tokens the cache holds over all live requests (num_pages = ceil(max_tokens / page_size)
            unless num_pages is given).  With neither, the pool is sized from the GPU's memory as the
            reference does (infer/src/scheduler/cuda/core/construction.rs:131-203): what is free once the
            weights are loaded, less a headroom of (1 - mem_fraction_static) of the whole memory, divided by
            the bytes of a page over all layers; never more than max_slots requests of max_request_tokens
            (default: the model's positions) can hold, since pages are not shared.
        max_slots: requests that run at a time.  None: as many requests of max_request_tokens (default: the model's
            positions) as the cache's tokens, given or sized from memory, hold; at least 4 and at most 128, as the
            reference's server picks them (infer/src/main.rs:782-855).
        max_request_tokens: longest single request (default: min(model's positions, cache capacity)).
        cuda_graph: replay steps of single decoded tokens from captured HIP graphs (the reference captures
            its decode path per batch size: infer/src/model/qwen3/batch_decode.rs:1691-1730).
        product_table: a table (or the path of its file) that says which kernel runs each matrix product at each
            row count, measured for this model's widths (`bench.py --tune-products`); without one, the rules that
            were measured at the Qwen3-4B, 8B and 32B widths decide.  The table is the process's, not this engine's.
        weight_tiles: hold every bfloat16 projection weight a second time in the layout that the few-rows
            kernels stream fastest (decode steps about a tenth faster, twice the weight memory).  Default:
            yes if both copies together stay under a third of the GPU's memory.
        """
        self.device = _device(device)
        self.dtype = parse_dtype(dtype)
        self.spec = spec
        if product_table is not None:
            ops.load_product_table(product_table)
        if weight_tiles is None:
            held = sum(t.numel() * t.element_size() for t in tensors.values() if t.dim() == 2)
            weight_tiles = 2 * held * 3 <= torch.cuda.get_device_properties(self.device).total_memory
        self.rt = Runtime(device=self.device, act_dtype=self.dtype,
                          weight_tiles=bool(weight_tiles) and self.dtype == torch.bfloat16)
        self.model = build_model(spec, tensors, self.rt)
        needs, readers = self.model.cache_needs()
        self.kv_bytes_per_token = cache_bytes_per_token(needs, self.dtype)
        if max_slots is None:
            longest = min(max_request_tokens or spec.max_positions, spec.max_positions)
            if num_pages is not None or max_tokens is not None:
                holds = num_pages * page_size if num_pages is not None else int(max_tokens)
            else:
                free, total = torch.cuda.mem_get_info(self.device)
                holds = page_size * pages_for_memory(free, total, mem_fraction_static, self.kv_bytes_per_token * page_size)
            max_slots = slots_for_tokens(holds, longest)
        if num_pages is None and max_tokens is None:
            longest = min(max_request_tokens or spec.max_positions, spec.max_positions)
            free, total = torch.cuda.mem_get_info(self.device)
            num_pages = pages_for_memory(free, total, mem_fraction_static, self.kv_bytes_per_token * page_size,
                                         reserved_bytes=max_slots * state_bytes_per_slot(needs),
                                         most_pages=max_slots * -(-longest // page_size))
            if num_pages < 1 and any(isinstance(n, PagedNeed) for n in needs):
                raise EngineError(f"no memory for the cache: {free / 2**30:.1f} GiB are free, the headroom of "
                                  f"{(1 - mem_fraction_static) * 100:.0f} % of {total / 2**30:.1f} GiB leaves less than "
                                  f"one page of {self.kv_bytes_per_token * page_size} bytes")
            num_pages = max(num_pages, 1)
        elif num_pages is None:
            num_pages = -(-int(max_tokens) // page_size)
        capacity = num_pages * page_size
        if max_request_tokens is None:
            max_request_tokens = min(spec.max_positions, capacity)
        self.cache = CacheManager(needs, page_size=page_size, num_pages=num_pages,
                                  max_slots=max_slots, max_request_tokens=max_request_tokens,
                                  device=self.device, dtype=self.dtype, readers=readers)
        self.page_size = page_size
        self.max_request_tokens = max_request_tokens
        # whatever a part keeps per position is made for the longest request now: no step, eager or captured, grows it
        self.model.prepare(max_request_tokens)
        self.steps_run = 0
        # the debugging dump of hidden states reads them on the host after every layer: such steps are not captured
        self.use_graphs = bool(cuda_graph) and self.model.graph_safe and os.environ.get(DEBUG_DUMP_ENV) is None
        self._graphs: dict = {}       # (rows, split cap) or a step shape -> (graph, input buffer, logits)
        self._shapes_seen: set = set()
        self.max_graphs = 64          # captured steps kept (each holds its activations)
        self.max_graph_logits_bytes = 64 << 20
        self._graph_pool = None
        self.graph_replays = 0

    # -- construction -----------------------------------------------------------------
    @classmethod
    def from_folder(cls, model_dir: str, *, dtype="bfloat16", device=None, **cache_args) -> "Engine":
        """A model folder (config.json + safetensors); the model class comes from config.json."""
        arch, config, stops = load_model_config(model_dir)
        spec = arch.recipe(config, stops)
        dev = _device(device)
        tensors = load_weights(model_dir, expected_checkpoint_tensors(spec), dev, parse_dtype(dtype))
        engine = cls(spec, tensors, dtype=dtype, device=dev, **cache_args)
        engine.config, engine.architecture = config, arch.name
        return engine

    @classmethod
    def from_config(cls, arch_name: str, config, *, seed: int = 0, std: float = 0.02,
                    norm_std: float = 0.0, dtype="bfloat16", device=None, **cache_args) -> "Engine":
        """Random weights drawn on the GPU from a configuration and a seed (no files)."""
        arch = detect_architecture({"architectures": [arch_name]})
        spec = arch.recipe(config, ())
        dev = _device(device)
        tensors = random_weights(spec, seed, std, norm_std, parse_dtype(dtype), device=dev)
        engine = cls(spec, tensors, dtype=dtype, device=dev, **cache_args)
        engine.config, engine.architecture = config, arch.name
        return engine

    # -- requests -----------------------------------------------------------------------
    def add_request(self, key) -> int:
        return self.cache.admit(key)

    def end_request(self, key) -> None:
        self.cache.release(key)

    def length(self, key) -> int:
        return self.cache.length(key)

    # -- the step -------------------------------------------------------------------------
    @torch.no_grad()
    def step(self, entries, borrow_logits: bool = False) -> torch.Tensor:
        """Run one packed step; returns float32 logits [wanted, vocab] on the GPU.

        Raises `OutOfPages` (nothing changed) if the cache cannot take all entries.
        borrow_logits: the caller is done with the logits before it calls `step` again (everything that reads
        them is queued on this stream by then, as the scheduler's sampling is), so a captured step may hand out
        the buffer that its next replay writes instead of a copy of it.
        """
        entries = [e if isinstance(e, StepEntry) else StepEntry(*e) for e in entries]
        if not entries:
            raise ValueError("a step needs at least one entry")
        for e in entries:
            if not self.cache.is_live(e.request):
                raise EngineError(f"request {e.request!r} is not live; add_request it first")
        before = {e.request: self.cache.length(e.request) for e in entries}
        decode_only = self.use_graphs and all(len(e.tokens) == 1 for e in entries)
        shape_key = None if decode_only or not self.use_graphs else self._repeated_shape(entries, before)
        batch = None
        if shape_key is not None:
            pass    # packed inside the captured path, like a decode step
        elif not decode_only:
            batch = build_step_batch(entries, self.cache.slot_of.__getitem__, self.cache.length,
                                     self.spec.vocab_size, self.device)
        else:   # the packing inside the captured path checks the token ids; on an error the lengths are rolled back
            if len({e.request for e in entries}) != len(entries):
                raise ValueError("a request appears twice in one step")
            for e in entries:
                if any(int(w) != 0 for w in e.want):
                    raise ValueError(f"wanted place outside the one token of request {e.request!r}")
                if not isinstance(e.tokens[0], DeviceToken) and not 0 <= int(e.tokens[0]) < self.spec.vocab_size:
                    raise ValueError(f"token id {e.tokens[0]} of request {e.request!r} is outside the vocabulary "
                                     f"(size {self.spec.vocab_size})")
        self.cache.append([(e.request, len(e.tokens)) for e in entries])
        saved_state = None
        try:
            # a mixer with state of its own overwrites it while the step runs: keep what a failed step must leave
            saved_state = self.cache.snapshot_state([e.request for e in entries])
            self.cache.sync_tables()
            if decode_only:
                logits = self._decode_step_graphed(entries, before, borrow_logits)
            elif shape_key is not None:
                logits = self._step_graphed(shape_key, entries, before, borrow_logits)
            else:
                logits = self.model.forward(batch, self.cache)
        except Exception:
            for key, n in before.items():
                self.cache.truncate(key, n)
            self.cache.restore_state(saved_state)
            raise
        for e in entries:
            self.cache.trim_windows(e.request)
        self.steps_run += 1
        return logits

    # -- captured decode steps ----------------------------------------------------------------
    def _decode_step_graphed(self, entries, before, borrow: bool = False) -> torch.Tensor:
        """A step of single decoded tokens through a HIP graph captured for its number of rows.

        The graph computes the logits of every row; the wanted ones are picked afterwards.  What
        varies from step to step (token ids, positions, slots) is copied into the graph's fixed
        input buffer; block tables are device tensors at fixed addresses already.  Launch shapes
        are part of the graph, so a graph is keyed by the number of rows and by what the parts say
        their launches depend on beside it (`Part.decode_launch_class`: the split-KV factor of the
        attention, which follows the longest context).
        """
        rows = len(entries)
        max_kv = max(before[e.request] for e in entries) + 1
        key = (rows, self.model.decode_launch_class(rows, max_kv))
        all_rows = [StepEntry(e.request, e.tokens, [0]) for e in entries]
        length_before = before.__getitem__
        rec = self._graphs.pop(key, None)
        if rec is None:
            static = torch.empty(packed_size(rows, rows, rows), dtype=torch.int32, device=self.device)
            batch = build_step_batch(all_rows, self.cache.slot_of.__getitem__, length_before,
                                     self.spec.vocab_size, self.device, into=static)
            batch.kv_splits = None
            logits = self.model.forward(batch, self.cache)   # this step's result, and the warm-up
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            if self._graph_pool is None:
                self._graph_pool = torch.cuda.graph_pool_handle()
            with torch.cuda.graph(graph, pool=self._graph_pool):
                static_logits = self.model.forward(batch, self.cache)
            rec = (graph, static, static_logits)
            while len(self._graphs) >= self.max_graphs:      # the least recently used goes
                self._graphs.pop(next(iter(self._graphs)))
        else:
            graph, static, static_logits = rec
            build_step_batch(all_rows, self.cache.slot_of.__getitem__, length_before,
                             self.spec.vocab_size, self.device, into=static)
            graph.replay()
            self.graph_replays += 1
            logits = static_logits if borrow else static_logits.clone()
        self._graphs[key] = rec    # most recently used last
        wanted = [i for i, e in enumerate(entries) for _ in e.want]
        if wanted == list(range(rows)):
            return logits
        return logits[torch.tensor(wanted, dtype=torch.long, device=self.device)]

    def warm_up(self, batch_sizes=None, max_context: int | None = None) -> int:
        """Capture the graphs of decode steps before the first request, so that no step of serving pays for an
        eager pass and a capture: for every batch size asked for (default: `decode_warmup_sizes` of the slots, the
        reference's schedule) and every class of context length up to `max_context` (default: the longest request)
        that changes a launch.  The reference does this when its scheduler starts
        (infer/src/scheduler/cuda/core/warmup.rs:11-160).  Runs dummy requests of token 0 through `step`, which
        leaves nothing behind but the graphs and pages that were written and given back.  Returns how many graphs
        were captured; batch sizes and contexts that the slots or the pool cannot hold are left out."""
        if not self.use_graphs:
            return 0
        sizes = sorted({int(b) for b in (batch_sizes or decode_warmup_sizes(self.cache.max_slots))
                        if 0 < int(b) <= self.cache.free_slot_count})
        longest = max(1, min(int(max_context or self.max_request_tokens), self.max_request_tokens))
        contexts = sorted({1, longest} | {1 << k for k in range(1, longest.bit_length()) if (1 << k) <= longest})
        wanted = {}
        for rows in sizes:
            for context in contexts:
                wanted.setdefault((rows, self.model.decode_launch_class(rows, context)), context)
        todo = [(key, context) for key, context in wanted.items() if key not in self._graphs]
        self.max_graphs = max(self.max_graphs, len(self._graphs) + len(todo) + 16)
        captured = 0
        for (rows, _), context in todo:
            names = [("__warm_up__", i) for i in range(rows)]
            try:
                for name in names:
                    self.add_request(name)
                if context > 1:
                    self.cache.append([(names[0], context - 1)])    # bookkeeping only: the keys are whatever the pages hold
                self.step([StepEntry(name, [0], [0]) for name in names])
                captured += 1
            except OutOfPages:
                pass        # the pool does not hold this context beside the other rows: serving will not see it either
            finally:
                for name in names:
                    if self.cache.is_live(name):
                        self.end_request(name)
        return captured

    def tune_products(self, rows=None, path: str | None = None, say=None) -> dict:
        """Measure, for the widths of this model, which kernel runs each of its matrix products fastest at each row
        count (`arle_amd.kernels.tune`), take the table in and, with `path`, write it there for the next start
        (`product_table=path`).  The reference tunes its library products when its scheduler starts
        (infer/src/scheduler/cuda/core/warmup.rs:100-131).  Half a minute to a minute and a half for a model of a
        few billion parameters; captured steps are dropped, since they hold the old choices."""
        from ..kernels import tune

        found = {}
        for part in self.model.parts:
            for name, n, k, fused, consumer in (part.products() if hasattr(part, "products") else []):
                found.setdefault((n, k, fused), (name, n, k, fused, consumer))
        products = [p + ((tune.HEAD_ROWS,) if p[0] == "head" else ()) for p in found.values()]
        table, _ = tune.tune_products(products, device=self.device, tiled=self.rt.weight_tiles, say=say, rows=rows)
        ops.load_product_table(table)
        if path:
            tune.write_table(path, table)
        self._graphs.clear()
        self._shapes_seen.clear()
        self._graph_pool = None
        return table

    # -- captured steps of any shape ---------------------------------------------------------------
    def _repeated_shape(self, entries, before):
        """Key of this step's launch shape if a step of the same shape has been seen before, else None.

        Every launch of a step is fixed by the lengths of its entries (in order), by how many logits are
        wanted, and by the cap that the longest context puts on the split-KV factor of its short entries.
        Serving repeats shapes (equal portions of a long prompt; the same decoded tokens beside them), and
        for a small step the host needs longer to launch the kernels one by one than the GPU to run them:
        from its second occurrence on a shape is run from a captured graph.
        """
        lens = tuple(len(e.tokens) for e in entries)
        if not lens or min(lens) == 0:
            return None
        wanted = sum(len(e.want) for e in entries)
        if wanted * self.spec.vocab_size * 4 > self.max_graph_logits_bytes:
            return None     # a captured step keeps its logits buffer for good
        max_kv = max(before[e.request] + len(e.tokens) for e in entries)
        key = (lens, wanted, ops.decode_split_cap(max_kv))
        if key in self._graphs:
            return key
        if len(self._shapes_seen) > 4096:
            self._shapes_seen.clear()
        seen = key in self._shapes_seen
        self._shapes_seen.add(key)
        return key if seen else None

    def _step_graphed(self, key, entries, before, borrow: bool = False) -> torch.Tensor:
        """A step whose shape repeats, through a HIP graph captured for that shape (see _repeated_shape).

        As for decode steps, what varies (token ids, positions, slots, wanted rows) travels in the graph's
        fixed input buffer.  The least recently used graph goes when there are too many.
        """
        length_before = before.__getitem__
        slot_of = self.cache.slot_of.__getitem__
        rec = self._graphs.pop(key, None)
        if rec is None:
            tokens, wanted = sum(key[0]), key[1]
            static = torch.empty(packed_size(tokens, len(entries), wanted), dtype=torch.int32, device=self.device)
            batch = build_step_batch(entries, slot_of, length_before, self.spec.vocab_size, self.device, into=static)
            logits = self.model.forward(batch, self.cache)   # this step's result, and the warm-up
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            if self._graph_pool is None:
                self._graph_pool = torch.cuda.graph_pool_handle()
            with torch.cuda.graph(graph, pool=self._graph_pool):
                static_logits = self.model.forward(batch, self.cache)
            rec = (graph, static, static_logits)
            while len(self._graphs) >= self.max_graphs:
                self._graphs.pop(next(iter(self._graphs)))
        else:
            graph, static, static_logits = rec
            build_step_batch(entries, slot_of, length_before, self.spec.vocab_size, self.device, into=static)
            graph.replay()
            self.graph_replays += 1
            logits = static_logits if borrow else static_logits.clone()
        self._graphs[key] = rec    # most recently used last
        return logits
