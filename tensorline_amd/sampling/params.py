"""Request options and per-request statistics, with the reference's names and defaults
(tensorline/engine.py:24-39)."""
from __future__ import annotations

from dataclasses import dataclass, field


@dataclass
class SamplingParams:
    max_tokens: int = 128
    temperature: float = 0.0            # <= 0: greedy
    top_p: float = 1.0
    stop_token_ids: set[int] = field(default_factory=set)   # empty: the model's end-of-sequence ids
    seed: int | None = None             # draws depend on (seed, position) only, not on batch mates


@dataclass
class GenStats:
    prompt_tokens: int = 0
    completion_tokens: int = 0
    cached_tokens: int = 0              # prompt tokens served from the prefix cache
    ttft_s: float = 0.0
    total_s: float = 0.0
    finish_reason: str = "length"       # "length" | "stop" | "abort"
