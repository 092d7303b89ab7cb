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

from ..kernels import ops
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
        if logits.shape[0] != len(rows):
            raise ValueError("one sampling row per row of logits is needed")
        if not rows:
            return [], None
        if any(p.has_penalties() and gen for p, _, _, gen in rows):
            logits = logits.clone()
            self._penalise(logits, rows)
        chosen = self._choose(logits, rows)
        if not any(p.logprobs for p, _, _, _ in rows):
            return chosen.tolist(), None
        logprobs = ops.token_logprobs(logits, chosen)
        return chosen.tolist(), logprobs.tolist()

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
        dev = torch.from_numpy(packed).to(self.device)
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
