"""The engine loop: schedule, run one step, sample, accept, finish.

One call of :meth:`InferenceEngine.step` is one iteration of the reference's scheduler loop
(tensorline/batch_engine.py:535-567 with ``_step`` 369-393): build the plan, run all planned
tokens as one batch through the step function, sample one token for every request whose plan
reached the end of its tokens, append or finish.  It runs on the caller's thread.

Steady decoding overlaps the host with the GPU (the reference's overlap scheduler,
batch_engine.py:478-533): a step in which every running request decodes one token is left *in
flight*, its sampled tokens still on the device.  If at the next call all of those requests
surely go on (none reaches its token or length limit with the token in flight, nobody waits to be
admitted, pages are there), the next step is queued first, taking its token ids from the device,
and only then are the earlier step's tokens read and accepted: the GPU runs step t + 1 while the
host handles step t.  A request that step t turns out to end (a stop token) has a wasted row in
step t + 1, which is ignored; its pages go back at once, which is safe because whatever uses them
next is queued behind step t + 1.  Anything else (admissions, prompt portions, a limit reached,
no page) takes the plain path: read, accept, schedule, run.
"""
from __future__ import annotations

import itertools
import random
import time
from dataclasses import dataclass

from tensorline_amd.cache.manager import CacheManager
from tensorline_amd.engine.batch import StepEntry
from tensorline_amd.engine.metrics import EngineMetrics
from tensorline_amd.engine.runner import ModelRunner
from tensorline_amd.engine.scheduler import Request, Scheduler
from tensorline_amd.sampling.params import GenStats, SamplingParams
from tensorline_amd.sampling.sampler import Sampler


@dataclass
class _InFlight:
    """A step that was queued and whose sampled tokens have not been read yet."""
    sampled: list                     # the requests a token was sampled for, in row order
    tokens: object                    # their tokens: an int32 tensor on the device
    decode_only: bool                 # every planned request decoded one token, and each was sampled
    host: object = None               # pinned host copy of the tokens, on its way since the step was queued
    landed: object = None             # event recorded behind that copy


class InferenceEngine:
    def __init__(self, model, cache: CacheManager, *, max_num_seqs: int = 64, max_batched_tokens: int = 2048,
                 max_model_len: int = 4096, default_stops: set[int] | None = None, runner: ModelRunner | None = None,
                 overlap: bool = True):
        self.model, self.cache = model, cache
        self.runner = runner or ModelRunner(model, cache)
        self.scheduler = Scheduler(cache, max_num_seqs, max_batched_tokens, max_model_len)
        self.sampler = Sampler(model.device)
        self.default_stops = set(default_stops or ())
        self._ids = itertools.count()
        self._seed_source = random.Random(0)
        # counters and distributions (reference: batch_engine.py:119-125, metrics.py:37-43)
        self.steps = 0
        self.overlapped_steps = 0
        self.metrics = EngineMetrics()
        self.overlap = bool(overlap)
        self._inflight: _InFlight | None = None
        self._token_buffers: list = []                    # two pinned buffers: the step in flight and the one before
        self._flip = 0

    # ---- requests ------------------------------------------------------------------------------
    def add_request(self, prompt_tokens: list[int], params: SamplingParams | None = None,
                    stats: GenStats | None = None) -> Request:
        params = params or SamplingParams()
        params.validate()
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
        return self.scheduler.has_work() or self._inflight is not None

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
        (request, None) for every request that ended (its ``error`` is set if it failed).  The
        tokens of a decode step may come with the next call (see the module's text)."""
        events: list[tuple[Request, int | None]] = []
        prev = self._inflight
        if prev is not None and self._all_go_on(prev):
            nxt = self._launch_ahead(prev)
            if nxt is not None:
                self._inflight = nxt
                self.overlapped_steps += 1
                self._retire(prev, events)               # the GPU is busy with the step just queued
                return events
        if prev is not None:
            self._inflight = None
            self._retire(prev, events)
        sched = self.scheduler
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
        decode_only = len(sampled) == len(plan) and all(n == 1 for _, n in plan)
        flight = self._launch(plan, entries, sampled, decode_only, None, 0)
        if self.overlap and decode_only and hasattr(self.sampler, "sample_device"):
            self._inflight = flight                      # read at the next call, perhaps behind the next step
        else:
            self._retire(flight, events)
        return events

    def drain(self) -> list[tuple[Request, int | None]]:
        """Read and accept the tokens of the step in flight, if there is one, without queueing another."""
        events: list[tuple[Request, int | None]] = []
        if self._inflight is not None:
            flight, self._inflight = self._inflight, None
            self._retire(flight, events)
        return events

    def _launch(self, plan, entries, sampled, decode_only, token_source, ahead: int) -> _InFlight:
        """Queue one step and the sampling of its tokens; nothing is awaited.  ``ahead``: how many of a
        request's generated tokens are not on the host yet (the index of its random draw moves on)."""
        sched = self.scheduler
        try:
            logits = self.runner.step(entries, token_source) if token_source is not None else self.runner.step(entries)
            args = (logits, [r.params.temperature for r in sampled], [r.params.top_p for r in sampled],
                    [r.seed for r in sampled], [r.num_generated + ahead for r in sampled])
            device_side = getattr(self.sampler, "sample_device", None)
            toks = device_side(*args) if device_side is not None else self.sampler.sample(*args)
        except Exception as e:
            self._inflight = None
            for req in sched.fail_all(e):
                self._count(req)
            raise
        self.steps += 1
        self.metrics.batch_size.observe(len(plan))
        sched.computed(plan)
        flight = _InFlight(sampled, toks, decode_only)
        if getattr(toks, "is_cuda", False):
            # The copy to the host is queued now, behind this step and before whatever is queued next:
            # reading it later waits for this step only, not for a step queued after it.
            import torch
            n = toks.numel()
            if len(self._token_buffers) < 2 or self._token_buffers[0].numel() < n:
                size = max(n, self.scheduler.max_num_seqs)
                self._token_buffers = [torch.empty(size, dtype=torch.int32, pin_memory=True) for _ in range(2)]
            self._flip ^= 1
            flight.host = self._token_buffers[self._flip][:n]
            flight.host.copy_(toks, non_blocking=True)
            flight.landed = torch.cuda.Event()
            flight.landed.record()
        return flight

    def _retire(self, flight: _InFlight, events: list) -> None:
        """Read a step's tokens (this waits for the step) and accept them."""
        sched = self.scheduler
        if flight.landed is not None:
            flight.landed.synchronize()
            toks = flight.host.tolist()
        else:
            toks = flight.tokens.tolist() if hasattr(flight.tokens, "tolist") else list(flight.tokens)
        now = time.perf_counter()
        for req, tok in zip(flight.sampled, toks):
            if req.done:                                 # ended while this step was in flight: a wasted row
                continue
            first = req.num_generated == 0 and req.stats.ttft_s == 0.0
            if sched.accept(req, int(tok), now):
                self.metrics.tokens_generated += 1
                events.append((req, int(tok)))
            if first:
                self.metrics.ttft_s.observe(req.stats.ttft_s)
            if req.done:
                self._count(req)
                events.append((req, None))

    def _all_go_on(self, flight: _InFlight) -> bool:
        """Whether the step after ``flight`` is known without its tokens: the same requests, each one
        token further.  Only a stop token can still end one of them, which costs a wasted row."""
        sched = self.scheduler
        if not (self.overlap and flight.decode_only) or sched.running != flight.sampled:
            return False
        if sched.waiting and len(sched.running) < sched.max_num_seqs:
            return False                                  # somebody may be admitted: that needs the whole picture
        for req in flight.sampled:
            # the token in flight is appended when it is read; there must be room for one more after it
            if req.done or req.num_generated + 2 > req.params.max_tokens or len(req.tokens) + 2 > sched.max_model_len:
                return False
        return True

    def _launch_ahead(self, prev: _InFlight) -> _InFlight | None:
        """Queue the step after ``prev`` with ``prev``'s tokens taken from the device; None if a page is missing."""
        reqs = prev.sampled
        for req in reqs:                                  # the token in flight sits at position num_computed
            if not self.cache.grow(req.rid, req.num_computed + 1):
                return None
        plan = [(req, 1) for req in reqs]
        entries = [StepEntry(req.rid, [0], req.num_computed, [0]) for req in reqs]
        return self._launch(plan, entries, reqs, True, prev.tokens, 1)

    def run_until_done(self) -> None:
        while self.has_work():
            self.step()

    def counters(self) -> dict:
        """Totals since the engine started, and the distributions of time to first token, whole
        request time (seconds) and sequences per step."""
        s, m = self.scheduler, self.metrics.as_dict()
        return {"steps": self.steps, "preemptions": s.preemptions, "max_running_seen": s.max_running_seen,
                "prompt_tokens_total": s.prompt_tokens_total, "prefix_hit_tokens": s.prefix_hit_tokens,
                "graph_replays": getattr(self.runner, "graph_replays", 0), "overlapped_steps": self.overlapped_steps, **m}
