"""Choosing the next token of every row of a step's logits.

All rows greedy and without penalties: one argmax kernel.  Otherwise: penalties on the
logits (repetition, frequency, presence over the tokens generated so far), then per row
softmax(logits / T), min-p, top-k, top-p and an inverse-CDF draw in token order.

The uniform number of a draw is a pure function of (seed, request's own draw index), so a
request's tokens do not depend on which other requests share its steps.  The reference
draws one number per request per step from a shared generator in slot order
(infer/src/model/qwen3/forward.rs:458-508), which ties results to batch composition; that
is not kept.
"""
from __future__ import annotations

import numpy as np
import torch

from ..engine.batch import DeviceToken
from ..kernels import ops
from ..kernels.upload import upload
from .params import SamplingParams

_MASK = (1 << 64) - 1


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    z = x
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def uniform(seed: int, index: int) -> float:
    """The index-th uniform number in [0, 1) of a request whose seed is `seed` (24 bits, exact in float32)."""
    return (_splitmix64(_splitmix64(seed & _MASK) ^ (index & _MASK)) >> 40) / float(1 << 24)


class Chosen:
    """The tokens that a step's sampling kernels chose, still on the GPU: handed to the next step as they are
    (`feed`), and on their way into pinned host memory by a copy queued right behind the kernels, before anything
    else is launched, so that reading them (`tokens`, `logprobs`) waits for the step that chose them and not for
    the step launched after it.  (The reference reads its argmax back asynchronously into a ring of pinned
    buffers: infer/src/model/qwen3/batch_decode.rs:728-774.  A copy stream of its own was tried here and taken
    out: while its wait for the step sits in a second hardware queue, every kernel of the step takes 0.7 us longer
    to start, 0.23 ms a step of the Qwen3-4B shape.)"""

    def __init__(self, token_tensor, logprob_tensor=None, read_back: bool = True):
        self.token_tensor = token_tensor       # int32 [rows]
        self.logprob_tensor = logprob_tensor   # float32 [rows] or None
        self._tokens = self._logprobs = self._arrived = None
        self._host = []
        if read_back and token_tensor.is_cuda:
            for t in (token_tensor, logprob_tensor):
                if t is not None:
                    self._host.append(torch.empty(t.shape, dtype=t.dtype, pin_memory=True).copy_(t, non_blocking=True))
            self._arrived = torch.cuda.Event()
            self._arrived.record()

    def feed(self, row: int) -> DeviceToken:
        return DeviceToken(self.token_tensor, row)

    def _read(self) -> None:
        if self._tokens is not None:
            return
        if self._arrived is None:
            self._tokens = self.token_tensor.tolist()
            self._logprobs = None if self.logprob_tensor is None else self.logprob_tensor.tolist()
            return
        self._arrived.synchronize()
        self._tokens = self._host[0].tolist()
        self._logprobs = self._host[1].tolist() if len(self._host) > 1 else None

    def tokens(self) -> list:
        self._read()
        return self._tokens

    def logprobs(self):
        self._read()
        return self._logprobs


class Sampler:
    def __init__(self, device):
        self.device = device

    def sample(self, logits: torch.Tensor, rows) -> list:
        """rows: one (SamplingParams, seed, draw_index, generated_tokens) per row of `logits`."""
        return self.sample_with_logprobs(logits, rows)[0]

    def sample_with_logprobs(self, logits: torch.Tensor, rows):
        """(token ids, log-probabilities): the second is None unless a row asks for `logprobs`; then it holds,
        for every row, log softmax(logits)[token] of the (penalised) logits, before temperature and truncation
        (for a greedy row: the reference's -log(sum exp(x - max)), crates/cuda-kernels/csrc/misc/sampling.cu:252-317)."""
        if not rows:
            if logits.shape[0] != 0:
                raise ValueError("one sampling row per row of logits is needed")
            return [], None
        chosen = self.choose(logits, rows)
        return chosen.tokens(), chosen.logprobs()

    def choose(self, logits: torch.Tensor, rows) -> Chosen:
        """As sample_with_logprobs, but nothing is read back: the kernels are queued and the result stays on the GPU."""
        if logits.shape[0] != len(rows):
            raise ValueError("one sampling row per row of logits is needed")
        if any(p.has_penalties() and gen for p, _, _, gen in rows):
            logits = logits.clone()
            self._penalise(logits, rows)
        chosen = self._choose(logits, rows)
        if not any(p.logprobs for p, _, _, _ in rows):
            return Chosen(chosen)
        return Chosen(chosen, ops.token_logprobs(logits, chosen))

    def _choose(self, logits: torch.Tensor, rows) -> torch.Tensor:
        if all(p.is_greedy() for p, _, _, _ in rows):
            return ops.argmax_rows(logits)
        # one host->device copy for the five per-row arrays (top_k travels as the bits of an int32)
        n, vocab = len(rows), logits.shape[1]
        packed = np.empty((5, n), dtype=np.float32)
        packed[0] = [p.temperature for p, _, _, _ in rows]
        packed[1] = [p.top_p for p, _, _, _ in rows]
        packed[2] = [p.min_p for p, _, _, _ in rows]
        packed[3] = [uniform(seed, idx) for _, seed, idx, _ in rows]
        packed[4].view(np.int32)[:] = [p.top_k for p, _, _, _ in rows]
        dev = upload(packed, self.device)      # queued: the host does not wait for the step that made the logits
        out = ops.sample_rows(logits, dev[0], dev[4].view(torch.int32), dev[1], dev[2], dev[3],
                              use_top_k=any(0 < p.top_k < vocab for p, _, _, _ in rows),
                              use_top_p=any(p.top_p < 1.0 for p, _, _, _ in rows))
        return out

    def _penalise(self, logits, rows) -> None:
        indptr, toks, counts = [0], [], []
        for p, _, _, generated in rows:
            if p.has_penalties():
                seen: dict = {}
                for t in generated:
                    seen[t] = seen.get(t, 0) + 1
                toks.extend(seen.keys())
                counts.extend(seen.values())
            indptr.append(len(toks))
        i32 = lambda vals: torch.tensor(vals, dtype=torch.int32, device=self.device)
        f32 = lambda vals: torch.tensor(vals, dtype=torch.float32, device=self.device)
        ops.apply_penalties(logits, i32(indptr), i32(toks), i32(counts),
                            f32([p.repetition_penalty for p, _, _, _ in rows]),
                            f32([p.frequency_penalty for p, _, _, _ in rows]),
                            f32([p.presence_penalty for p, _, _, _ in rows]))
