"""What the engine counts while it runs: totals, and distributions of time to first token, of a
request's whole time and of the number of sequences in a step.

The quantities and the bucket bounds are the reference's (tensorline/metrics.py:9-43; observed at
batch_engine.py:363,383,398); its Prometheus text is a server's business and has no counterpart
here.  A distribution keeps a count per bucket (bounds are upper limits, a last bucket takes
everything above), the sum, and the smallest and largest value, and estimates a quantile from the
buckets.  Everything is updated from the engine's own thread.
"""
from __future__ import annotations

import bisect
from dataclasses import dataclass, field

LATENCY_BOUNDS_S = (0.01, 0.025, 0.05, 0.1, 0.25, 0.5, 1, 2.5, 5, 10, 30, 60)
BATCH_BOUNDS = (1, 2, 4, 8, 16, 32, 64, 128)


class Distribution:
    def __init__(self, bounds):
        self.bounds = tuple(float(b) for b in bounds)
        if list(self.bounds) != sorted(set(self.bounds)):
            raise ValueError("bucket bounds must increase")
        self.counts = [0] * (len(self.bounds) + 1)
        self.count, self.total = 0, 0.0
        self.smallest, self.largest = float("inf"), float("-inf")

    def observe(self, value: float) -> None:
        value = float(value)
        self.counts[bisect.bisect_left(self.bounds, value)] += 1      # a value on a bound belongs to that bucket
        self.count += 1
        self.total += value
        self.smallest, self.largest = min(self.smallest, value), max(self.largest, value)

    @property
    def mean(self) -> float:
        return self.total / self.count if self.count else 0.0

    def quantile(self, q: float) -> float:
        """The value below which a share ``q`` of the observations lies, taken linearly inside the
        bucket it falls into and never outside what was observed."""
        if not self.count:
            return 0.0
        rank, seen = q * self.count, 0
        for i, c in enumerate(self.counts):
            if c and seen + c >= rank:
                lo = self.bounds[i - 1] if i > 0 else 0.0
                hi = self.bounds[i] if i < len(self.bounds) else self.largest
                lo, hi = max(lo, self.smallest), min(hi, self.largest)
                return lo + (hi - lo) * max(0.0, min(1.0, (rank - seen) / c))
            seen += c
        return self.largest

    def as_dict(self) -> dict:
        labels = [f"le_{b:g}" for b in self.bounds] + ["above"]
        return {"count": self.count, "sum": self.total, "mean": self.mean,
                "min": self.smallest if self.count else 0.0, "max": self.largest if self.count else 0.0,
                "p50": self.quantile(0.5), "p99": self.quantile(0.99),
                "buckets": dict(zip(labels, self.counts))}


@dataclass
class EngineMetrics:
    ttft_s: Distribution = field(default_factory=lambda: Distribution(LATENCY_BOUNDS_S))
    e2e_s: Distribution = field(default_factory=lambda: Distribution(LATENCY_BOUNDS_S))
    batch_size: Distribution = field(default_factory=lambda: Distribution(BATCH_BOUNDS))
    tokens_generated: int = 0
    requests_finished: dict = field(default_factory=dict)          # finish reason -> count

    def finished(self, reason: str, total_s: float | None = None) -> None:
        self.requests_finished[reason] = self.requests_finished.get(reason, 0) + 1
        if total_s is not None:
            self.e2e_s.observe(total_s)

    def as_dict(self) -> dict:
        return {"tokens_generated": self.tokens_generated, "requests_finished": dict(self.requests_finished),
                "ttft_s": self.ttft_s.as_dict(), "e2e_s": self.e2e_s.as_dict(), "batch_size": self.batch_size.as_dict()}
