"""A model built from a ModelSpec: embedding, blocks run in schedule order, final norm, head.

Nothing here knows an architecture.  The forward pass of a packed step follows the
reference's order (infer/src/model/qwen3/prefill.rs:460-547): embed all rows, run the
layers, then norm and project only the rows whose logits are wanted
(infer/src/model/qwen3/batch_decode.rs:1519-1601 compacts them the same way).
"""
from __future__ import annotations

import os
import sys

from ..kernels import ops
from ..parts import base  # noqa: F401  (registries)
from ..parts import attention, block, embedding, feed_forward, norm, position  # noqa: F401  registers the stock parts
from ..parts.base import Runtime, build_part, expected_tensors, lookup
from ..parts.spec import ModelSpec


def expected_checkpoint_tensors(spec: ModelSpec) -> dict:
    """checkpoint tensor name -> WeightDecl over the whole model (a tied tensor appears once)."""
    out: dict = {}

    def merge(found: dict) -> None:
        for name, decl in found.items():
            if name in out and tuple(out[name].shape) != tuple(decl.shape):
                raise ValueError(f"tensor '{name}' is used with two shapes: {out[name].shape} and {decl.shape}")
            out.setdefault(name, decl)

    merge(expected_tensors("embedding", spec.embedding))
    for layer in spec.layers:
        if layer.mixer is not None:
            merge(expected_tensors("mixer", layer.mixer))
        if layer.feed_forward is not None:
            merge(expected_tensors("feed_forward", layer.feed_forward))
        for norm_spec in layer.norms.values():
            merge(expected_tensors("norm", norm_spec))
        for role, part_spec in layer.parts.values():
            merge(expected_tensors(role, part_spec))
    merge(expected_tensors("norm", spec.final_norm))
    merge(expected_tensors("head", spec.head))
    return out


def declared_cache_needs(spec: ModelSpec) -> list:
    """The cache need of every schedule entry as its mixer's class declares it from the spec alone (no
    weights, no GPU): what a shape summary and a memory plan are made from."""
    needs = []
    for entry in spec.schedule:
        if entry.cache_from is not None:
            needs.append(None)
        else:
            mixer = spec.layers[entry.layer].mixer
            needs.append(None if mixer is None else lookup("mixer", mixer.kind).declare_cache(mixer.params))
    return needs


def kv_cache_bytes_per_token(spec: ModelSpec, act_dtype) -> int:
    """Bytes of cache one token takes over all layers; for Qwen3 2 * layers * kv_heads * head_dim * element size
    (infer/src/model/qwen3/forward.rs:777-783)."""
    from ..cache.manager import cache_bytes_per_token

    return cache_bytes_per_token(declared_cache_needs(spec), act_dtype)


DEBUG_DUMP_ENV = "ARLE_AMD_DEBUG_DUMP"


def debug_dump(residual, delta, label: str) -> None:
    """With ARLE_AMD_DEBUG_DUMP set: one line to stderr about the hidden state of the step's last row after every
    schedule entry (first and last values, minimum, maximum, root mean square, NaN or infinity anywhere), as the
    reference prints with INFER_DEBUG_DUMP (infer/src/model/common.rs:85-124).  Synchronises; steps are then not
    captured."""
    row = residual[-1].float()
    if delta is not None:
        row = row + (delta.float().sum(0) if delta.dim() == 3 else delta.float())[-1]
    row = row.cpu()
    fmt = lambda vals: "[" + ", ".join(f"{v:+.5f}" for v in vals.tolist()) + "]"
    print(f"[debug-dump] {label}: head={fmt(row[:8])} tail={fmt(row[-4:])} min={float(row.min()):.4f} "
          f"max={float(row.max()):.4f} rms={float(row.pow(2).mean().sqrt()):.4f} nan={bool(row.isnan().any())} "
          f"inf={bool(row.isinf().any())}", file=sys.stderr, flush=True)


class DecoderModel:
    def __init__(self, spec: ModelSpec, fetch, rt: Runtime):
        spec.validate()
        self.spec = spec
        self.rt = rt
        self.embedding = build_part("embedding", spec.embedding, fetch, rt)
        self.blocks = []
        self._extra_parts = []
        for layer in spec.layers:
            mixer = build_part("mixer", layer.mixer, fetch, rt) if layer.mixer is not None else None
            ffn = build_part("feed_forward", layer.feed_forward, fetch, rt) if layer.feed_forward is not None else None
            norms = {role: build_part("norm", s, fetch, rt) for role, s in layer.norms.items()}
            if layer.parts:     # an arrangement with further parts takes them as a fourth argument
                extra = {name: build_part(role, s, fetch, rt) for name, (role, s) in layer.parts.items()}
                self._extra_parts.extend(extra.values())
                self.blocks.append(lookup("block", layer.block)(mixer, ffn, norms, extra))
            else:
                self.blocks.append(lookup("block", layer.block)(mixer, ffn, norms))
        self.schedule = list(spec.schedule)
        self.final_norm = build_part("norm", spec.final_norm, fetch, rt)
        self.head = build_part("head", spec.head, fetch, rt)
        parts = [self.embedding, self.final_norm, self.head, *self._extra_parts]
        for b in self.blocks:
            parts += [p for p in (b.mixer, b.feed_forward) if p is not None] + list(getattr(b, "norms", {}).values())
        self.parts = parts
        self.graph_safe = all(getattr(p, "graph_safe", False) for p in parts)

    def prepare(self, max_positions: int) -> None:
        """Every part gets to size what it keeps per position for the longest request, before the first step."""
        for part in self.parts:
            prepare = getattr(part, "prepare", None)
            if prepare is not None:
                prepare(max_positions)

    def decode_launch_class(self, rows: int, max_context: int) -> tuple:
        """What the launches of a step of `rows` single decoded tokens depend on beyond `rows`, over all parts (the
        distinct answers of `Part.decode_launch_class`, in a fixed order)."""
        found = set()
        for part in self.parts:
            ask = getattr(part, "decode_launch_class", None)
            answer = ask(rows, max_context) if ask is not None else None
            if answer is not None:
                found.add(answer)
        return tuple(sorted(found, key=repr))

    def cache_needs(self):
        """(need of every schedule entry that owns a cache, {reader entry -> owner entry})."""
        needs, readers = [], {}
        for i, entry in enumerate(self.schedule):
            if entry.cache_from is not None:
                needs.append(None)
                readers[i] = entry.cache_from
            else:
                mixer = self.blocks[entry.layer].mixer
                needs.append(mixer.cache_need() if mixer is not None else None)
        return needs, readers

    def forward(self, batch, cache):
        """Logits float32 [len(batch.want_rows), vocab] of one packed step."""
        # every pass over the layers gets a name of its own (a pass that is being captured into a graph too: its
        # first layer has to plan inside the graph): parts that prepare something once a step key it with this
        batch.plan_token = ops.new_plan_token()
        residual = self.embedding.forward(batch.token_ids)
        delta = None
        dump = os.environ.get(DEBUG_DUMP_ENV) is not None
        if dump:
            debug_dump(residual, None, "embedding")
        for i, entry in enumerate(self.schedule):
            residual, delta = self.blocks[entry.layer].forward(residual, delta, batch, cache.view(i))
            if dump:
                debug_dump(residual, delta, f"schedule entry {i} (layer {entry.layer})")
        wanted = self.final_norm.add_norm(residual, delta, rows=batch.want_rows)
        return self.head.forward(wanted)


def build_model(spec: ModelSpec, tensors: dict, rt: Runtime) -> DecoderModel:
    return DecoderModel(spec, tensors.__getitem__, rt)
