"""Sampling parameters, with the reference's names, defaults and greedy rule
(infer/src/sampler.rs:15-84)."""
from __future__ import annotations

from dataclasses import dataclass, field


@dataclass
class SamplingParams:
    temperature: float = 0.0          # 0 = greedy (argmax)
    top_k: int = -1                   # -1 = off
    top_p: float = 1.0                # 1.0 = off
    min_p: float = 0.0                # 0 = off; keep p >= min_p * p_max
    repetition_penalty: float = 1.0   # over generated tokens; 1.0 = off
    frequency_penalty: float = 0.0
    presence_penalty: float = 0.0
    ignore_eos: bool = False
    stop_token_ids: list = field(default_factory=list)
    seed: int | None = None           # None = the engine's seed
    max_new_tokens: int | None = None
    logprobs: bool = False            # report log softmax(logits)[chosen token] of every generated token

    def is_greedy(self) -> bool:
        """(temperature <= 0 or top_k == 1) and no stochastic filter (infer/src/sampler.rs:82-84)."""
        return (self.temperature <= 0.0 or self.top_k == 1) and self.top_p >= 1.0 and self.min_p <= 0.0

    def has_penalties(self) -> bool:
        return (self.repetition_penalty != 1.0 or self.frequency_penalty != 0.0
                or self.presence_penalty != 0.0)
