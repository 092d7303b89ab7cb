"""Registries of parts by role, the runtime handed to every part, and the part interfaces.

Roles: "embedding", "norm", "position", "mixer", "feed_forward", "block", "head".
A part class declares the parameters it needs (`declare_weights`) and any parts nested
in it (`children`), is built from its sizes, its tensors and its children, and never
learns which model it is in.

Interfaces (T = tokens of the packed step, H = hidden size, A = activation dtype):

* norm          `forward(x[T,W]) -> A[T,W]`;  `add_norm(residual f32[T,H], delta | None,
                rows=None) -> A[rows or T, H]` adds the delta into the residual (in place) first.
                A delta is A[T,H], or a float32 stack [S,T,H] of partial sums to be added in the order
                of S (what a matrix product with K split over workgroups leaves behind).
* position      `fused_rotary() -> (cos, sin, rotary_dim) | None`;  `apply(q, k, positions)` in place.
* mixer         `cache_need() -> PagedNeed | StateNeed | None` (and, so that a model's cache can be sized
                from its description alone, the class method `declare_cache(params)` with the same answer);
                `forward(x A[T,H], batch: StepBatch, cache_view) -> delta`.
* feed_forward  `forward(x A[T,H]) -> delta`.
* block         `forward(residual f32[T,H], delta | None, batch, cache_view) -> (residual, delta)`;
                the returned delta is what the next block (or the final norm) still has to add.
* embedding     `forward(token_ids i32[T]) -> f32[T,H]`.
* head          `forward(x A[R,H]) -> f32[R,V]`.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .spec import PartSpec, Rows, WeightDecl, tensor_name

ROLES = ("embedding", "norm", "position", "mixer", "feed_forward", "block", "head")
_REGISTRY: dict = {role: {} for role in ROLES}


class UnknownPart(KeyError):
    pass


def register(role: str, kind: str):
    """Class decorator: make `kind` buildable wherever a spec asks for it in `role`."""
    if role not in _REGISTRY:
        raise ValueError(f"unknown role {role!r}; roles are {ROLES}")

    def deco(cls):
        _REGISTRY[role][kind] = cls
        cls.role, cls.kind = role, kind
        return cls

    return deco


def lookup(role: str, kind: str):
    try:
        return _REGISTRY[role][kind]
    except KeyError:
        known = ", ".join(sorted(_REGISTRY.get(role, {}))) or "none"
        raise UnknownPart(f"no {role} part named {kind!r} is registered (known: {known})") from None


@dataclass
class Runtime:
    """Where and in which precision a model runs."""

    device: torch.device
    act_dtype: torch.dtype  # torch.bfloat16 (serving) or torch.float32 (true 32-bit path)
    # keep a second copy of every bfloat16 projection weight as operand tiles, the layout that the few-rows
    # kernels stream fastest (twice the weight memory; the library keeps reading the rows)
    weight_tiles: bool = False

    @property
    def is_f32(self) -> bool:
        return self.act_dtype == torch.float32


class Part:
    role = ""
    kind = ""
    # True if forward() launches the same kernels with the same arguments for every step of a given
    # shape, reading whatever varies (positions, slots, lengths) from GPU memory: only then may the
    # engine replay the part from a captured graph.
    graph_safe = False

    @classmethod
    def declare_weights(cls, params: dict) -> dict:
        """parameter name -> WeightDecl."""
        return {}

    @classmethod
    def children(cls, params: dict) -> dict:
        """child name -> (role, PartSpec) of parts nested in this one."""
        return {}

    @classmethod
    def declare_cache(cls, params: dict):
        """What a mixer of these sizes keeps between steps (PagedNeed | StateNeed | None), known without building
        it.  A mixer that only answers `cache_need()` on a built instance is sized from the built model."""
        return None

    def __init__(self, params: dict, tensors: dict, rt: Runtime, children: dict | None = None):
        self.params = params
        self.rt = rt
        self.child_parts = dict(children or {})

    def products(self) -> list:
        """The bfloat16 matrix products this part runs, for a tuner that measures which kernel runs each fastest:
        [(name, N, K, with the gate|up activation, "norm" if the result goes into a residual add and norm or a
        kernel that adds a stack of partial products itself, else None)]."""
        return []

    def decode_launch_class(self, rows: int, max_context: int):
        """What of a step of `rows` single decoded tokens, the longest of whose contexts is `max_context` tokens,
        the launches of this part depend on beyond `rows` (a hashable value; None: nothing).  Two such steps with
        equal answers from every part launch the same kernels with the same arguments, so one captured graph
        serves both."""
        return None

    def prepare(self, max_positions: int) -> None:
        """Called by the engine once the longest request is known, before any step runs or is captured: whatever
        a part keeps that grows with the position (a table of angles, slopes, a window of taps) is made for
        `max_positions` positions here, so that no step has to allocate.  The default hands the call on to the
        parts nested in this one."""
        for child in getattr(self, "child_parts", {}).values():
            prepare = getattr(child, "prepare", None)
            if prepare is not None:
                prepare(max_positions)


def expected_tensors(role: str, spec: PartSpec) -> dict:
    """checkpoint tensor name -> WeightDecl for a part and everything nested in it."""
    cls = lookup(role, spec.kind)
    out = {}
    for pname, decl in cls.declare_weights(spec.params).items():
        if pname not in spec.weights:
            raise ValueError(f"{role} part {spec.kind!r}: no tensor name given for parameter {pname!r}")
        source = spec.weights[pname]
        if isinstance(source, Rows):
            # the parameter is some rows of a larger checkpoint tensor: that tensor is what the folder must hold
            if not decl.shape or decl.shape[0] != source.stop - source.start:
                raise ValueError(f"{role} part {spec.kind!r}: parameter {pname!r} has {decl.shape[0] if decl.shape else 0} "
                                 f"rows, the recipe gives it rows {source.start}:{source.stop} of '{source.tensor}'")
            decl = WeightDecl((source.of, *decl.shape[1:]), decl.init)
        name = tensor_name(source)
        if name in out and tuple(out[name].shape) != tuple(decl.shape):
            raise ValueError(f"tensor '{name}' is used with two shapes: {out[name].shape} and {decl.shape}")
        out[name] = decl
    for _, (child_role, child_spec) in cls.children(spec.params).items():
        out.update(expected_tensors(child_role, child_spec))
    return out


def build_part(role: str, spec: PartSpec, fetch, rt: Runtime):
    """Construct a part; `fetch(tensor_name)` returns the loaded tensor."""
    cls = lookup(role, spec.kind)
    tensors = {}
    for pname in cls.declare_weights(spec.params):
        source = spec.weights[pname]
        whole = fetch(tensor_name(source))
        tensors[pname] = whole[source.start:source.stop] if isinstance(source, Rows) else whole
    kids = {name: build_part(r, s, fetch, rt) for name, (r, s) in cls.children(spec.params).items()}
    return cls(spec.params, tensors, rt, kids)


__all__ = ["register", "lookup", "Runtime", "Part", "expected_tensors", "build_part", "WeightDecl",
           "PartSpec", "Rows", "UnknownPart", "ROLES"]
