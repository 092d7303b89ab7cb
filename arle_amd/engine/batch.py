"""A packed step: the rows of several requests side by side, and the arrays kernels read.

A step is a list of entries (request, its next tokens, wanted places).  Rows are laid out
in the order given; a decoded token is simply an entry of one token.  The reference builds
the same arrays for its kernels -- positions, qo_indptr, kv_indptr/indices
(crates/cuda-kernels/src/tilelang.rs:424-618,703-819) -- except that block tables live on
the GPU for the life of a request here and are not flattened per step.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch


@dataclass
class StepEntry:
    request: object          # key of a live request
    tokens: list             # its next token ids (>= 1)
    want: list = field(default_factory=list)  # places among `tokens` whose logits are wanted


@dataclass
class Segment:
    request: object
    slot: int
    start: int    # position of the first token of this portion
    length: int
    row0: int     # first row of the portion in the packed step


@dataclass
class StepBatch:
    num_tokens: int
    segments: list
    max_position: int
    max_qlen: int                # longest segment
    min_qlen: int                # shortest segment
    token_ids: torch.Tensor      # int32 [T]
    positions: torch.Tensor      # int32 [T]  absolute position of each row in its request
    slot_of_token: torch.Tensor  # int32 [T]  row of the block tables / state buffers
    want_rows: torch.Tensor      # int32 [R]  rows whose logits are returned, in entry/want order
    seg_row0: torch.Tensor       # int32 [S+1] first row of each segment (qo_indptr)
    seg_slot: torch.Tensor       # int32 [S]
    seg_start: torch.Tensor      # int32 [S]  position of a segment's first row
    host: dict                   # the same arrays as numpy, for parts that plan on the host
    kv_splits: int | None = None  # split-KV factor fixed by the caller (a captured graph), else chosen per call


def packed_size(num_tokens: int, num_segments: int, num_wanted: int) -> int:
    """int32 elements that the device arrays of a step take together."""
    return 3 * num_tokens + num_wanted + (num_segments + 1) + 2 * num_segments


def build_step_batch(entries, slot_of, length_of, vocab_size: int, device, into=None) -> StepBatch:
    """Check a step's entries and lay them out.

    slot_of(request) -> slot;  length_of(request) -> tokens cached before this step.
    into: an int32 device buffer of exactly `packed_size(...)` elements to fill instead of a
    fresh one (a captured graph reads its inputs from fixed addresses).
    """
    if not entries:
        raise ValueError("a step needs at least one entry")
    seen = set()
    segments, ids, pos, slots, want_rows = [], [], [], [], []
    row = 0
    for e in entries:
        if e.request in seen:
            raise ValueError(f"request {e.request!r} appears twice in one step")
        seen.add(e.request)
        n = len(e.tokens)
        if n == 0:
            raise ValueError(f"request {e.request!r} brings no tokens")
        slot, start = slot_of(e.request), length_of(e.request)
        for t in e.tokens:
            if not 0 <= int(t) < vocab_size:
                raise ValueError(f"token id {t} of request {e.request!r} is outside the vocabulary "
                                 f"(size {vocab_size})")
        for w in e.want:
            if not 0 <= int(w) < n:
                raise ValueError(f"wanted place {w} of request {e.request!r} is outside its {n} tokens")
            want_rows.append(row + int(w))
        segments.append(Segment(e.request, slot, start, n, row))
        ids.extend(int(t) for t in e.tokens)
        pos.extend(range(start, start + n))
        slots.extend([slot] * n)
        row += n
    host = {
        "token_ids": np.asarray(ids, dtype=np.int32),
        "positions": np.asarray(pos, dtype=np.int32),
        "slot_of_token": np.asarray(slots, dtype=np.int32),
        "want_rows": np.asarray(want_rows, dtype=np.int32),
        "seg_row0": np.asarray([s.row0 for s in segments] + [row], dtype=np.int32),
        "seg_slot": np.asarray([s.slot for s in segments], dtype=np.int32),
        "seg_start": np.asarray([s.start for s in segments], dtype=np.int32),
    }
    # one host->device copy for all arrays
    order = list(host)
    sizes = [host[k].size for k in order]
    flat = torch.from_numpy(np.concatenate([host[k] for k in order]))
    if into is None:
        packed = flat.to(device, non_blocking=False)
    else:
        if into.numel() != flat.numel():
            raise ValueError("the fixed step buffer does not fit this step")
        into.copy_(flat)
        packed = into
    dev, off = {}, 0
    for k, n in zip(order, sizes):
        dev[k] = packed[off:off + n]
        off += n
    return StepBatch(num_tokens=row, segments=segments, max_position=max(pos),
                     max_qlen=max(s.length for s in segments), min_qlen=min(s.length for s in segments),
                     host=host, **dev)
