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

from ..cache import native
from ..kernels.upload import staging_for, upload


@dataclass(frozen=True)
class DeviceToken:
    """A token that the host does not know yet: element `row` of an int32 tensor on the GPU, which a sampling
    kernel of the step before wrote (or will have written when this step's kernels run: same stream).  As the one
    token of an entry it lets the next decode step be launched before the last one's tokens are read back, as the
    reference hands its argmax output to the next step on the device (infer/src/model/qwen3/batch_decode.rs:683-774)."""
    source: object
    row: int


@dataclass
class StepEntry:
    request: object          # key of a live request
    tokens: list             # its next token ids (>= 1), or [DeviceToken]
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
    single_segments: int = 0     # segments of one token (decoded tokens)
    kv_splits: int | None = None  # split-KV factor fixed by the caller (a captured graph), else chosen per call
    plan_token: int = 0          # names one pass over the layers (set by the model): what parts plan once a pass
    max_portion_kv: int = 0      # longest context (cached + new) among the segments of more than one token; 0: none


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
    segments, row = [], 0
    fed = []     # (row of the step, DeviceToken): token ids that come from GPU memory
    for e in entries:
        if e.request in seen:
            raise ValueError(f"request {e.request!r} appears twice in one step")
        seen.add(e.request)
        if len(e.tokens) == 0:
            raise ValueError(f"request {e.request!r} brings no tokens")
        if len(e.tokens) == 1 and isinstance(e.tokens[0], DeviceToken):
            fed.append((row, e.tokens[0]))
        segments.append(Segment(e.request, slot_of(e.request), length_of(e.request), len(e.tokens), row))
        row += len(e.tokens)
    # the arrays themselves are laid out by the native runtime core, which also checks ids and places;
    # its inputs go over in one int32 array: slots, starts, token counts, want counts, tokens, wants
    S = len(segments)
    staged = [s.slot for s in segments]
    staged += [s.start for s in segments]
    staged += [s.length for s in segments]
    staged += [len(e.want) for e in entries]
    if fed:
        device_rows = {r for r, _ in fed}
        for seg, e in zip(segments, entries):
            staged += [0] if seg.row0 in device_rows and seg.length == 1 else e.tokens   # 0 until the GPU fills it in
    else:
        for e in entries:
            staged += e.tokens
    for e in entries:
        staged += e.want
    try:
        wide = np.array(staged)
        if wide.dtype.kind not in "iu":     # a float would be cut to an integer without a word, a bool read as 0 or 1
            raise TypeError
        wide = wide.astype(np.int64)
    except (TypeError, ValueError, OverflowError):
        raise ValueError("token ids and wanted places are integers (a DeviceToken only as the one token of an "
                         "entry)") from None
    np.clip(wide, -1, 2**31 - 1, out=wide)     # what is out of range stays out of range
    inputs = wide.astype(np.int32)
    num_wanted = inputs.size - 4 * S - row
    base = inputs.ctypes.data
    at = lambda elements: base + 4 * elements
    slot_p, start_p, ntok_p, nwant_p, tokens_p, wants_p = at(0), at(S), at(2 * S), at(3 * S), at(4 * S), at(4 * S + row)
    flat_np = np.empty(packed_size(row, S, num_wanted), dtype=np.int32)
    meta, where = native.int_array(6), native.int_array(2)
    code = native.lib().arle_pack_step(S, slot_p, start_p, ntok_p, tokens_p, nwant_p, wants_p, int(vocab_size),
                                       flat_np.ctypes.data, flat_np.size, meta, where)
    if code == 1:
        e = entries[where[0]]
        bad = next(t for t in e.tokens if not 0 <= int(t) < vocab_size)
        raise ValueError(f"token id {bad} of request {e.request!r} is outside the vocabulary (size {vocab_size})")
    if code == 2:
        e = entries[where[0]]
        bad = next(w for w in e.want if not 0 <= int(w) < len(e.tokens))
        raise ValueError(f"wanted place {bad} of request {e.request!r} is outside its {len(e.tokens)} tokens")
    if code != 0:
        raise ValueError(f"the step could not be packed (code {code})")
    sizes = [row, row, row, num_wanted, S + 1, S, S]
    order = ["token_ids", "positions", "slot_of_token", "want_rows", "seg_row0", "seg_slot", "seg_start"]
    host, off = {}, 0
    for k, n in zip(order, sizes):
        host[k] = flat_np[off:off + n]
        off += n
    # one host->device copy for all arrays, through pinned memory: the host does not wait for the stream
    if into is None:
        packed = upload(flat_np, device) if torch.device(device).type == "cuda" else torch.from_numpy(flat_np)
    else:
        if into.numel() != flat_np.size:
            raise ValueError("the fixed step buffer does not fit this step")
        staging_for(device).copy_into(into, flat_np)
        packed = into
    dev, off = {}, 0
    for k, n in zip(order, sizes):
        dev[k] = packed[off:off + n]
        off += n
    if fed:
        feed_device_tokens(dev["token_ids"], fed)
    return StepBatch(num_tokens=row, segments=segments, max_position=meta[2], max_qlen=meta[3], min_qlen=meta[4],
                     single_segments=meta[5],
                     max_portion_kv=max((s.start + s.length for s in segments if s.length > 1), default=0),
                     host=host, **dev)


def feed_device_tokens(token_ids: torch.Tensor, fed) -> None:
    """token_ids[row] = source[source_row] for every (row, DeviceToken(source, source_row)), on the GPU."""
    by_source: dict = {}
    for row, tok in fed:
        by_source.setdefault(id(tok.source), (tok.source, [], []))
        by_source[id(tok.source)][1].append(row)
        by_source[id(tok.source)][2].append(int(tok.row))
    for source, rows, source_rows in by_source.values():
        if source.device != token_ids.device or source.dim() != 1:
            raise ValueError("a DeviceToken names a one-dimensional tensor on the engine's GPU")
        if min(source_rows) < 0 or max(source_rows) >= source.numel():
            raise ValueError("a DeviceToken names a row outside its tensor")
        n = len(rows)
        if rows == list(range(rows[0], rows[0] + n)) and source_rows == list(range(source_rows[0], source_rows[0] + n)):
            token_ids[rows[0]:rows[0] + n].copy_(source[source_rows[0]:source_rows[0] + n])     # the usual case: one copy
            continue
        index = upload(np.array([rows, source_rows], dtype=np.int32), token_ids.device).long()
        token_ids.index_copy_(0, index[0], source.index_select(0, index[1]).to(torch.int32))

