"""Continuous batching: which request runs how many tokens in the next step.

The decisions are those of the reference's ``BatchEngine._schedule`` (tensorline/batch_engine.py:
314-356), on host data only:

1. Running requests are served first, oldest first: one token when decoding, the next portion of
   the prompt otherwise, under one token budget for the whole step (``max_batched_tokens``).
2. When the cache has no page for a running request, the *newest* running request is preempted:
   its pages and state slot are given back, it returns to the front of the waiting queue and is
   later computed again from its first token, prompt and generated tokens alike (recompute
   preemption, batch_engine.py:292-298).  If the request that needs the page is itself the newest,
   it is the one preempted.
3. Waiting requests are admitted first-come-first-served while budget, ``max_num_seqs`` and pages
   allow; a prompt longer than the budget is admitted in portions.  A request that does not fit
   even when nothing else runs fails with an error instead of waiting forever.

Beyond the reference: a request that the pool can never hold, even alone, ends with
:class:`RequestError` instead of being admitted, preempting itself and being admitted again
forever (the reference only catches a first portion that does not fit, batch_engine.py:343-346).
It is refused when added if its prompt is too long already; it fails at (re)admission if its
prompt and generated tokens are; and it fails where it preempts itself while nothing else runs,
which is how a request that outgrows the pool in the middle of a later portion or while decoding
shows, whatever ``max_batched_tokens`` is.
"""
from __future__ import annotations

import time
from collections import deque
from dataclasses import dataclass, field

from tensorline_amd.cache.manager import CacheManager
from tensorline_amd.sampling.params import GenStats, SamplingParams


class RequestError(RuntimeError):
    pass


@dataclass(eq=False)
class Request:
    rid: int
    prompt_len: int
    tokens: list[int]                     # prompt, then generated tokens
    params: SamplingParams
    stops: set[int]
    stats: GenStats = field(default_factory=GenStats)
    t_submit: float = field(default_factory=time.perf_counter)
    num_computed: int = 0                 # tokens whose keys and values are cached
    seed: int = 0
    done: bool = False
    error: Exception | None = None
    admitted_before: bool = False

    @property
    def num_generated(self) -> int:
        return len(self.tokens) - self.prompt_len

    @property
    def output_tokens(self) -> list[int]:
        return self.tokens[self.prompt_len:]


class Scheduler:
    def __init__(self, cache: CacheManager, max_num_seqs: int = 64, max_batched_tokens: int = 2048,
                 max_model_len: int = 4096):
        if max_num_seqs > cache.max_requests:
            raise ValueError(f"max_num_seqs {max_num_seqs} exceeds the cache's {cache.max_requests} state slots")
        self.cache = cache
        self.max_num_seqs, self.max_batched_tokens, self.max_model_len = max_num_seqs, max_batched_tokens, max_model_len
        self.waiting: deque[Request] = deque()
        self.running: list[Request] = []
        self.failed: list[Request] = []        # requests that ended with an error in schedule()
        # counters (reference: batch_engine.py:119-125)
        self.preemptions = 0
        self.max_running_seen = 0
        self.prompt_tokens_total = 0
        self.prefix_hit_tokens = 0

    # ---- queue -------------------------------------------------------------------------------
    def add(self, req: Request) -> None:
        if req.prompt_len <= 0:
            raise ValueError("a request needs at least one prompt token")
        if req.prompt_len >= self.max_model_len:
            raise ValueError(f"prompt has {req.prompt_len} tokens; max_model_len is {self.max_model_len}")
        if not self.cache.can_ever_hold(req.prompt_len + 1, self.max_batched_tokens):
            raise RequestError(
                f"request does not fit in the KV cache: {req.prompt_len} prompt tokens need "
                f"{self.cache.pages_for(req.prompt_len + 1)} pages, the pool has {self.cache.num_blocks}")
        req.stats.prompt_tokens = req.prompt_len
        self.waiting.append(req)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    def abort(self, req: Request) -> bool:
        """Stop a request wherever it is; its pages go back (batch_engine.py:300-312)."""
        if req in self.running:
            self.running.remove(req)
        elif req in self.waiting:
            self.waiting.remove(req)
        else:
            return False
        self._release(req)
        req.done = True
        req.stats.finish_reason = "abort"
        return True

    # ---- pages -------------------------------------------------------------------------------
    def _release(self, req: Request) -> None:
        if self.cache.has_request(req.rid):
            self.cache.release(req.rid)

    def _preempt(self, req: Request) -> None:
        self.running.remove(req)
        self._release(req)
        req.num_computed = 0
        self.waiting.appendleft(req)
        self.preemptions += 1

    def _fail_unholdable(self, req: Request) -> None:
        """End a request (already out of both queues, its pages given back) that the pool cannot hold."""
        req.done = True
        req.error = RequestError(
            f"request does not fit in the KV cache: its {len(req.tokens)} tokens and the next one need "
            f"{self.cache.pages_for(len(req.tokens) + 1)} pages, the pool has {self.cache.num_blocks}")
        self.failed.append(req)

    # ---- the plan ----------------------------------------------------------------------------
    def schedule(self) -> list[tuple[Request, int]]:
        budget = self.max_batched_tokens
        plan: list[tuple[Request, int]] = []
        preempted: set[int] = set()
        for req in list(self.running):                       # oldest first
            if id(req) in preempted:                         # preempted earlier in this pass
                continue
            n = min(len(req.tokens) - req.num_computed, budget)
            if n <= 0:
                continue
            fits = True
            while not self.cache.grow(req.rid, req.num_computed + n):
                victim = self.running[-1]                    # the newest running request
                self._preempt(victim)
                preempted.add(id(victim))
                budget += sum(k for r, k in plan if r is victim)
                plan = [(r, k) for r, k in plan if r is not victim]
                if victim is req:
                    fits = False
                    if not self.running:                     # it was alone and the whole pool is too small
                        self._fail_unholdable(self.waiting.popleft())
                    break
            if fits:
                plan.append((req, n))
                budget -= n
        while self.waiting and budget > 0 and len(self.running) < self.max_num_seqs:
            req = self.waiting[0]
            if not self.cache.can_ever_hold(len(req.tokens) + 1, self.max_batched_tokens):
                self._fail_unholdable(self.waiting.popleft())    # grew past the pool before it was preempted
                continue
            if self.cache.add_request(req.rid) is None:
                break                                        # no state slot free
            req.num_computed = self.cache.match_prefix(req.rid, req.tokens)
            n = min(len(req.tokens) - req.num_computed, budget)
            if not self.cache.grow(req.rid, req.num_computed + n):
                self._release(req)                           # drop prefix references while it waits
                req.num_computed = 0
                if not self.running:                         # can never fit, even alone
                    self._fail_unholdable(self.waiting.popleft())
                    continue
                break                                        # wait for pages to come back
            self.waiting.popleft()
            self.running.append(req)
            if not req.admitted_before:                      # first admission, not a re-admission
                req.admitted_before = True
                req.stats.cached_tokens = req.num_computed
                self.prompt_tokens_total += req.prompt_len
                self.prefix_hit_tokens += req.num_computed
            plan.append((req, n))
            budget -= n
        self.max_running_seen = max(self.max_running_seen, len(self.running))
        return plan

    def computed(self, plan: list[tuple[Request, int]]) -> None:
        """After the step ran: count the tokens as cached, publish full pages for prefix sharing and
        give back pages a window has passed (batch_engine.py:387-389)."""
        for req, n in plan:
            req.num_computed += n
            self.cache.publish(req.rid, req.tokens, req.num_computed)
            self.cache.trim(req.rid, req.num_computed)

    # ---- accepting a sampled token -------------------------------------------------------------
    def accept(self, req: Request, tok: int, now: float | None = None) -> bool:
        """Append a sampled token or finish the request; returns True if the token was appended
        (batch_engine.py:395-406: a stop token ends the request and is neither kept nor emitted)."""
        now = time.perf_counter() if now is None else now
        if req.num_generated == 0 and req.stats.ttft_s == 0.0:
            req.stats.ttft_s = now - req.t_submit
        if tok in req.stops:
            self.finish(req, "stop", now)
            return False
        req.tokens.append(tok)
        if req.num_generated >= req.params.max_tokens or len(req.tokens) >= self.max_model_len:
            self.finish(req, "length", now)
        return True

    def finish(self, req: Request, reason: str, now: float | None = None) -> None:
        now = time.perf_counter() if now is None else now
        req.done = True
        req.stats.finish_reason = reason
        req.stats.completion_tokens = req.num_generated
        req.stats.total_s = now - req.t_submit
        if req in self.running:
            self.running.remove(req)
        self._release(req)

    def fail_all(self, error: Exception) -> list[Request]:
        """A step raised: every request in flight fails rather than hangs (batch_engine.py:568-576)."""
        out = self.running + list(self.waiting)
        for req in out:
            self._release(req)
            req.done = True
            req.error = error
        self.running.clear()
        self.waiting.clear()
        return out
