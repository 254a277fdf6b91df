"""Per-request sampling options, names and meanings as in the reference
(`SamplingParams`, include/inferx/scheduler/scheduler.h:19-65)."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List


@dataclass
class SamplingParams:
    max_tokens: int = 16            # cap on generated tokens; reaching it is a normal finish
    stop_tokens: List[int] = field(default_factory=list)  # any of these ends the sequence (and stays in the output)
    temperature: float = 0.0        # zero or below: greedy
    top_p: float = 1.0              # at or above 1: off
    top_k: int = 0                  # 0: off
    min_p: float = 0.0              # 0: off; else drop tokens below min_p * p_max
    presence_penalty: float = 0.0   # subtracted once from every generated token's logit
    frequency_penalty: float = 0.0  # subtracted per occurrence
    repetition_penalty: float = 1.0  # positive logits divided, negative multiplied
    min_tokens: int = 0             # stop tokens are masked for the first min_tokens generated tokens
    ignore_eos: bool = False
    seed: int = 0                   # fixes the draws of this request
    want_logprobs: bool = False     # report the chosen token's log-probability ...
    top_logprobs: int = 0           # ... and up to this many (at most 20) of the most probable alternatives

    def validate(self) -> None:
        if self.max_tokens <= 0:
            raise ValueError("max_tokens must be positive")
        if self.top_k < 0 or not 0.0 < self.top_p or self.min_p < 0 or self.min_p > 1:
            raise ValueError("top_k must be >= 0, top_p > 0 and min_p within [0, 1]")
        if not 0 <= self.top_logprobs <= 20:
            raise ValueError("top_logprobs must be between 0 and 20")
        if self.repetition_penalty <= 0:
            raise ValueError("repetition_penalty must be positive")

    @property
    def needs_penalties(self) -> bool:
        return self.presence_penalty != 0.0 or self.frequency_penalty != 0.0 or self.repetition_penalty != 1.0
