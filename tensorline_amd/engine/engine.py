"""The engine loop: schedule, run one step, sample, accept, finish.

One call of :meth:`InferenceEngine.step` is one iteration of the reference's scheduler loop
(tensorline/batch_engine.py:535-567 with ``_step`` 369-393): build the plan, run all planned
tokens as one batch through the step function, sample one token for every request whose plan
reached the end of its tokens, append or finish.  It runs on the caller's thread.
"""
from __future__ import annotations

import itertools
import random
import time

from tensorline_amd.cache.manager import CacheManager
from tensorline_amd.engine.batch import StepEntry
from tensorline_amd.engine.metrics import EngineMetrics
from tensorline_amd.engine.runner import ModelRunner
from tensorline_amd.engine.scheduler import Request, Scheduler
from tensorline_amd.sampling.params import GenStats, SamplingParams
from tensorline_amd.sampling.sampler import Sampler


class InferenceEngine:
    def __init__(self, model, cache: CacheManager, *, max_num_seqs: int = 64, max_batched_tokens: int = 2048,
                 max_model_len: int = 4096, default_stops: set[int] | None = None, runner: ModelRunner | None = None):
        self.model, self.cache = model, cache
        self.runner = runner or ModelRunner(model, cache)
        self.scheduler = Scheduler(cache, max_num_seqs, max_batched_tokens, max_model_len)
        self.sampler = Sampler(model.device)
        self.default_stops = set(default_stops or ())
        self._ids = itertools.count()
        self._seed_source = random.Random(0)
        # counters and distributions (reference: batch_engine.py:119-125, metrics.py:37-43)
        self.steps = 0
        self.metrics = EngineMetrics()

    # ---- requests ------------------------------------------------------------------------------
    def add_request(self, prompt_tokens: list[int], params: SamplingParams | None = None,
                    stats: GenStats | None = None) -> Request:
        params = params or SamplingParams()
        toks = [int(t) for t in prompt_tokens]
        V = self.model.vocab_size
        if any(t < 0 or t >= V for t in toks):
            raise ValueError(f"prompt holds a token id outside [0, {V})")
        seed = params.seed if params.seed is not None else self._seed_source.getrandbits(63)
        req = Request(next(self._ids), len(toks), toks, params, set(params.stop_token_ids) or set(self.default_stops),
                      stats or GenStats(), seed=seed)
        self.scheduler.add(req)
        return req

    def abort(self, req: Request) -> None:
        if self.scheduler.abort(req):
            self._count(req)

    def has_work(self) -> bool:
        return self.scheduler.has_work()

    @property
    def tokens_generated(self) -> int:
        return self.metrics.tokens_generated

    @property
    def requests_finished(self) -> dict:
        return self.metrics.requests_finished

    def _count(self, req: Request) -> None:
        """A request ended: by its reason, and its whole time if it ran to a stop or its length."""
        reason = "error" if req.error is not None else req.stats.finish_reason
        self.metrics.finished(reason, req.stats.total_s if reason in ("stop", "length") else None)

    # ---- one iteration -------------------------------------------------------------------------
    def step(self) -> list[tuple[Request, int | None]]:
        """Returns the events of this iteration: (request, token) for every token appended and
        (request, None) for every request that ended (its ``error`` is set if it failed)."""
        sched = self.scheduler
        events: list[tuple[Request, int | None]] = []
        plan = sched.schedule()
        for req in sched.failed:
            self._count(req)
            events.append((req, None))
        sched.failed.clear()
        if not plan:
            return events
        entries, sampled = [], []
        for req, n in plan:
            end = req.num_computed + n
            want = [n - 1] if end == len(req.tokens) else []
            entries.append(StepEntry(req.rid, req.tokens[req.num_computed:end], req.num_computed, want))
            if want:
                sampled.append(req)
        try:
            logits = self.runner.step(entries)
            toks = self.sampler.sample(
                logits, [r.params.temperature for r in sampled], [r.params.top_p for r in sampled],
                [r.seed for r in sampled], [r.num_generated for r in sampled])
        except Exception as e:
            for req in sched.fail_all(e):
                self._count(req)
                events.append((req, None))
            raise
        self.steps += 1
        self.metrics.batch_size.observe(len(plan))
        sched.computed(plan)
        now = time.perf_counter()
        for req, tok in zip(sampled, toks):
            first = req.num_generated == 0 and req.stats.ttft_s == 0.0
            if sched.accept(req, int(tok), now):
                self.metrics.tokens_generated += 1
                events.append((req, int(tok)))
            if first:
                self.metrics.ttft_s.observe(req.stats.ttft_s)
            if req.done:
                self._count(req)
                events.append((req, None))
        return events

    def run_until_done(self) -> None:
        while self.has_work():
            self.step()

    def counters(self) -> dict:
        """Totals since the engine started, and the distributions of time to first token, whole
        request time (seconds) and sequences per step."""
        s, m = self.scheduler, self.metrics.as_dict()
        return {"steps": self.steps, "preemptions": s.preemptions, "max_running_seen": s.max_running_seen,
                "prompt_tokens_total": s.prompt_tokens_total, "prefix_hit_tokens": s.prefix_hit_tokens,
                "graph_replays": getattr(self.runner, "graph_replays", 0), **m}
