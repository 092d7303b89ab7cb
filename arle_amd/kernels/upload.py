"""Small arrays from the host to the GPU without making the host wait.

A copy from ordinary host memory makes the host wait until everything queued on the stream before it has run,
the model's step before included; from pinned memory it is queued like a kernel and the host goes on, which is
what lets the next step be prepared and launched while the last one still runs.  The reference uploads its
per-step metadata from pinned staging buffers for the same reason (infer/src/model/qwen3/batch_decode.rs:2462-2541).
"""
from __future__ import annotations

import numpy as np
import torch


class PinnedStaging:
    """A few pinned buffers used in turn, each with an event that says when its last copy has run, so that none is
    rewritten while the GPU may still read it."""

    def __init__(self, slots: int = 8):
        self.buffers = [None] * slots
        self.events = [None] * slots
        self.turn = 0

    def copy_into(self, into: torch.Tensor, values: np.ndarray) -> None:
        """into (on the GPU, contiguous, 4-byte elements) = values (int32 or float32, as many elements)."""
        if values.dtype not in (np.int32, np.float32) or into.element_size() != 4 or not into.is_contiguous():
            raise ValueError("staged copies carry contiguous arrays of 4-byte elements")
        if into.numel() != values.size:
            raise ValueError(f"the copy's target holds {into.numel()} elements, the values are {values.size}")
        i = self.turn
        self.turn = (self.turn + 1) % len(self.buffers)
        if self.events[i] is not None:
            self.events[i].synchronize()
        n = values.size
        if self.buffers[i] is None or self.buffers[i].numel() < n:
            self.buffers[i] = torch.empty(max(n, 1024), dtype=torch.int32, pin_memory=True)
        self.buffers[i].numpy()[:n] = values.reshape(-1).view(np.int32)
        into.view(torch.int32).view(-1).copy_(self.buffers[i][:n], non_blocking=True)
        if self.events[i] is None:
            self.events[i] = torch.cuda.Event()
        self.events[i].record()


_staging: dict = {}


def staging_for(device) -> PinnedStaging:
    key = str(device)
    if key not in _staging:
        _staging[key] = PinnedStaging()
    return _staging[key]


def upload(values: np.ndarray, device) -> torch.Tensor:
    """A new tensor on the GPU with these int32 or float32 values, queued on the current stream."""
    values = np.ascontiguousarray(values)
    out = torch.empty(values.shape, dtype=torch.int32 if values.dtype == np.int32 else torch.float32, device=device)
    if values.size:
        staging_for(device).copy_into(out, values)
    return out
