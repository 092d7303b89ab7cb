"""The description of a model as data: which parts, with which sizes, fed by which tensors.

An architecture's recipe (`arle_amd/models/*.py`) turns its typed configuration into a
`ModelSpec`.  Everything downstream of it -- the weight loader, the random-weight
writer, the cache manager and the step function -- reads only the spec, never the
architecture's name.

* `PartSpec`  one part: its kind (a name in the registry of its role), its sizes and
  constants, and the checkpoint tensor (or the rows of one: `Rows`) behind each of its parameters.
* `LayerSpec` one block: the arrangement and the mixer, feed-forward and norms in it.
  Layers need not be alike.
* `ModelSpec.schedule` the order in which layers run, as a list.  An entry may name a
  layer that another entry names too (shared weights, separate caches), or say that
  it reads the cache which an earlier entry writes (`cache_from`).
"""
from __future__ import annotations

from dataclasses import dataclass, field


@dataclass(frozen=True)
class WeightDecl:
    """What a part expects of one parameter: its shape and how random weights fill it."""

    shape: tuple
    init: str = "normal"  # a name known to weights.random_init: "normal" N(0, std), "ones" 1 + N(0, norm_std), "zeros", ...


@dataclass(frozen=True)
class Rows:
    """A parameter that is rows [start, stop) of a checkpoint tensor of `of` rows: what a recipe names in
    `PartSpec.weights` where the checkpoint stores several projections as one matrix (q|k|v, gate|up)."""

    tensor: str
    start: int
    stop: int
    of: int     # rows of the whole checkpoint tensor, so that its shape is known from the recipe alone

    def __post_init__(self):
        if not 0 <= self.start < self.stop <= self.of:
            raise ValueError(f"rows {self.start}:{self.stop} do not lie in a tensor of {self.of} rows")


def tensor_name(source) -> str:
    """The checkpoint tensor behind a `PartSpec.weights` value (a name, or `Rows` of a named tensor)."""
    return source.tensor if isinstance(source, Rows) else source


@dataclass
class PartSpec:
    kind: str
    params: dict = field(default_factory=dict)
    weights: dict = field(default_factory=dict)  # parameter name -> tensor name in the checkpoint, or Rows of one


@dataclass
class LayerSpec:
    """One block.  Most arrangements hold one mixer, one feed-forward and their norms; an arrangement may also do
    without one of the two (None), and may name further parts of any role in `parts`, which it is handed built
    (a second feed-forward beside the routed one, a gate, a norm of another kind)."""

    block: str                          # arrangement, a name in the "block" registry
    mixer: PartSpec | None = None
    feed_forward: PartSpec | None = None
    norms: dict = field(default_factory=dict)   # role in the arrangement -> PartSpec of a norm
    parts: dict = field(default_factory=dict)   # name -> (role, PartSpec) of further parts of the arrangement


@dataclass(frozen=True)
class ScheduleEntry:
    layer: int                     # index into ModelSpec.layers
    cache_from: int | None = None  # index of an earlier schedule entry whose cache is read


@dataclass
class ModelSpec:
    hidden_size: int
    vocab_size: int
    max_positions: int
    embedding: PartSpec
    layers: list
    schedule: list
    final_norm: PartSpec
    head: PartSpec
    stop_token_ids: tuple = ()

    def validate(self) -> None:
        for i, entry in enumerate(self.schedule):
            if not 0 <= entry.layer < len(self.layers):
                raise ValueError(f"schedule entry {i} names layer {entry.layer}, which does not exist")
            if entry.cache_from is not None:
                if not 0 <= entry.cache_from < i:
                    raise ValueError(f"schedule entry {i} reads the cache of entry {entry.cache_from}, "
                                     "which does not run before it")
                if self.schedule[entry.cache_from].cache_from is not None:
                    raise ValueError(f"schedule entry {i} reads the cache of entry {entry.cache_from}, "
                                     "which owns no cache itself")
