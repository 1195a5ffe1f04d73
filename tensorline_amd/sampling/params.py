"""Request options and per-request statistics, with the reference's names and defaults
(tensorline/engine.py:24-39)."""
from __future__ import annotations

import math
from dataclasses import dataclass, field


@dataclass
class SamplingParams:
    max_tokens: int = 128
    temperature: float = 0.0            # <= 0: greedy
    top_p: float = 1.0
    stop_token_ids: set[int] = field(default_factory=set)   # empty: the model's end-of-sequence ids
    seed: int | None = None             # draws depend on (seed, position) only, not on batch mates

    def validate(self) -> None:
        """Refuse options no sampling rule is defined for: the keep-rule of top-p keeps nothing at
        top_p <= 0 (tensorline/engine.py:47-49 would divide by zero there), and a request generates
        at least one token."""
        if not (isinstance(self.max_tokens, int) and self.max_tokens >= 1):
            raise ValueError(f"max_tokens must be an integer of at least 1, not {self.max_tokens!r}")
        if not math.isfinite(self.temperature):
            raise ValueError(f"temperature must be a finite number (<= 0 is greedy), not {self.temperature!r}")
        if not (math.isfinite(self.top_p) and self.top_p > 0.0):
            raise ValueError(f"top_p must be above 0 (1 and more keep every token), not {self.top_p!r}")


@dataclass
class GenStats:
    prompt_tokens: int = 0
    completion_tokens: int = 0
    cached_tokens: int = 0              # prompt tokens served from the prefix cache
    ttft_s: float = 0.0
    total_s: float = 0.0
    finish_reason: str = "length"       # "length" | "stop" | "abort"
