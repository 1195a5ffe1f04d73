"""HIP-graph replay of pure decode steps.

A decode step at small batch is a few hundred short kernels; launching them one by one costs more
than running them.  A graph records the whole step once and replays it with one launch
(reference: ``CudaGraphDecoder``, tensorline/cuda_graphs.py:38-126).  Graphs need fixed shapes and
addresses, so:

* the batch is padded to a bucket (1, 2, 4, ... max_num_seqs), and the step's longest context is
  rounded up to a context bucket (4,096 keys, doubling up to the longest the engine allows); one
  graph per pair, captured at first use or ahead of time by ``warmup``.  What a context bucket
  fixes is the number of key splits decode attention launches and merges: a graph captured for
  the longest context would launch and merge hundreds of empty splits at short ones (measured at
  the 7B shape with a limit of 32,768 and 2,300 live keys: 3.37 instead of 3.21 ms per step);
* the page tables always have the full width ``max_blocks_per_seq``: the kernels walk a table only
  up to the sequence's length, so its width costs nothing but the copy;
* all index data of a step lives in one int32 device buffer per graph, filled by one copy;
* padding rows read and write only the scratch page and the scratch state slot;
* graphs share one memory pool, as only one replays at a time.

No memset is recorded into a graph: every buffer a kernel needs cleared is cleared by a kernel.
Steps that are not pure decode (prompt portions, mixed batches) run eagerly.
"""
from __future__ import annotations

from typing import Sequence

import numpy as np
import torch

from tensorline_amd.cache.manager import CacheManager
from tensorline_amd.engine.batch import StepEntry
from tensorline_amd.engine.runner import ModelRunner


class _Captured:
    def __init__(self, graph, dev, host, logits, packed):
        self.graph, self.dev, self.host, self.logits, self.packed = graph, dev, host, logits, packed
        # what the host buffer holds since the last replay: the requests of its rows and their
        # positions, so that the next token of the same requests only touches a few numbers
        self.rids: tuple | None = None
        self.admissions: tuple = ()
        self.starts: np.ndarray | None = None
        self.copied: torch.cuda.Event | None = None      # recorded after the last copy out of the host buffer


class GraphRunner(ModelRunner):
    def __init__(self, model, cache: CacheManager, max_batch: int, max_blocks_per_seq: int):
        super().__init__(model, cache)
        # batch sizes a graph exists for: the powers of two below max_batch, and max_batch itself
        self.batch_buckets = sorted({1 << k for k in range(max(max_batch - 1, 0).bit_length())} | {max_batch})
        self.max_blocks = max_blocks_per_seq
        self.fit_context = max_blocks_per_seq * cache.page_size   # eager steps split keys as the graphs do
        # longest contexts a graph exists for: 4,096 keys doubling, and the longest a request may reach
        self.context_buckets = sorted({c for c in (4096 << k for k in range(24)) if c < self.fit_context} | {self.fit_context})
        self.graphs: dict[tuple[int, int], _Captured] = {}      # (batch bucket, context bucket) -> graph
        self.graph_replays = 0
        self.pool = None
        self.side = None

    # ---- which steps replay ------------------------------------------------------------------
    def can_run(self, entries: Sequence[StepEntry]) -> bool:
        """Pure decode: one token per request, not the first, its logits wanted
        (tensorline/cuda_graphs.py:52-55)."""
        if not entries or len(entries) > self.batch_buckets[-1]:
            return False
        for e in entries:
            if len(e.tokens) != 1 or e.start <= 0 or list(e.want) != [0]:
                return False
            if -(-(e.start + 1) // self.cache.page_size) > self.max_blocks:
                return False
        return True

    def _bucket(self, n: int) -> int:
        for b in self.batch_buckets:
            if n <= b:
                return b
        raise ValueError(f"{n} exceeds the largest bucket {self.batch_buckets[-1]}")

    def _context_bucket(self, tokens: int) -> int:
        for c in self.context_buckets:
            if tokens <= c:
                return c
        raise ValueError(f"a context of {tokens} tokens exceeds the longest a graph is captured for, {self.context_buckets[-1]}")

    # ---- capture -------------------------------------------------------------------------------
    def _padding_batch(self, B: int):
        """A batch of B padding rows: defines the layout of the graph's buffer."""
        from tensorline_amd.engine.batch import pack_batch
        cache = self.cache
        ng = len(cache.groups)
        pad = StepEntry("pad", [0], 0, [0])
        tables = [[[cache.scratch_page] for _ in range(ng)]]
        packed = pack_batch([pad], tables, [cache.scratch_slot], cache.page_size, ng, cache.scratch_page,
                            self.model.vocab_size, pad_seqs=B, pad_nb=[self.max_blocks] * ng,
                            scratch_slot=cache.scratch_slot, vectors=self._vectors)
        return packed

    @torch.inference_mode()
    def _capture(self, B: int, C: int) -> _Captured:
        packed = self._padding_batch(B)
        packed.facts.max_context, packed.facts.fit_context = C, self.fit_context
        packed.facts.decode_only = True
        n = packed.data.size
        dev = torch.empty(n, dtype=torch.int32, device=self.device)
        host = torch.empty(n, dtype=torch.int32, pin_memory=True)
        host.numpy()[:] = packed.data
        dev.copy_(host)
        ctx, views = self.context(packed, dev)
        if self.pool is None:
            self.pool = torch.cuda.graph_pool_handle()
            self.side = torch.cuda.Stream(device=self.device)
        side = self.side
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):              # warm-up outside capture: lazy initialisations
            for _ in range(2):
                self.model.forward(ctx, views)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, pool=self.pool):
            logits = self.model.forward(ctx, views)
        cap = _Captured(g, dev, host, logits, packed)
        self.graphs[(B, C)] = cap
        return cap

    def warmup(self, max_context_tokens: int = 0) -> int:
        """Capture every batch bucket before serving, largest first, for contexts of up to
        ``max_context_tokens`` (at least the shortest context bucket), so that no request up to that
        length pays for a capture (tensorline/cuda_graphs.py:84-96); longer contexts capture at first
        use.  Captures touch only the scratch page."""
        upto = self._context_bucket(min(max(max_context_tokens, 1), self.fit_context))
        for C in (c for c in self.context_buckets if c <= upto):
            for B in reversed(self.batch_buckets):
                if (B, C) not in self.graphs:
                    self._capture(B, C)
        torch.cuda.synchronize()
        return len(self.graphs)

    def _advance(self, cap: _Captured, entries: Sequence[StepEntry]) -> bool:
        """The common case of steady decoding: the same requests in the same rows as the bucket's
        last replay, each one token further.  Then the buffer is brought up to date in place (token,
        position, cache row, and a page id where a request entered a new page) instead of being
        packed again.  False: not that case, nothing was touched."""
        cache = self.cache
        if cap.rids is None or len(cap.rids) != len(entries) or cache.has_windows:
            return False
        for rid, adm, e in zip(cap.rids, cap.admissions, entries):
            if e.rid != rid or cache.admission(rid) != adm:  # another request, or the same one admitted again
                return False
        n = len(entries)
        starts = np.fromiter((e.start for e in entries), np.int64, n)
        if not np.array_equal(starts, cap.starts + 1):
            return False
        toks = np.fromiter((e.tokens[0] for e in entries), np.int64, n)
        if toks.min() < 0 or toks.max() >= self.model.vocab_size:
            raise ValueError(f"token id outside [0, {self.model.vocab_size})")
        buf, off = cap.host.numpy(), cap.packed.offsets
        page = cache.page_size
        lp, within = starts // page, starts % page
        fresh = np.nonzero(within == 0)[0]                   # requests whose token opens a page
        rows = np.arange(n)
        for g in range(len(cache.groups)):
            o, size = off[f"tables{g}"]
            tables = buf[o:o + size].reshape(cap.packed.S, cap.packed.group_nb[g])
            for i in fresh:
                tab = cache.table_array(cap.rids[i], g)
                if len(tab) <= lp[i]:
                    raise ValueError(f"request {cap.rids[i]!r}: page table covers {len(tab) * page} tokens, "
                                     f"{starts[i] + 1} are needed")
                tables[i, lp[i]] = tab[lp[i]]
            pages = tables[rows, lp]
            if pages.min() < 0:
                raise ValueError("a token of this step lies on a page already given back")
            o, _ = off[f"slots{g}"]
            buf[o:o + n] = pages * page + within
        for name, vals in (("ids", toks), ("pos", starts), ("ctx_start", starts)):
            o, _ = off[name]
            buf[o:o + n] = vals
        cap.starts = starts
        return True

    # ---- one step ------------------------------------------------------------------------------
    @torch.inference_mode()
    def step(self, entries: Sequence[StepEntry], token_source: torch.Tensor | None = None) -> torch.Tensor:
        if not self.can_run(entries):
            return super().step(entries, token_source)
        n = len(entries)
        B, C = self._bucket(n), self._context_bucket(max(e.start for e in entries) + 1)
        cap = self.graphs.get((B, C)) or self._capture(B, C)
        ng = len(self.cache.groups)
        if cap.copied is not None:
            cap.copied.synchronize()       # the host buffer is read by a copy that does not block: wait before writing it again
        if not self._advance(cap, entries):
            packed = self.pack(entries, pad_seqs=B, pad_nb=[self.max_blocks] * ng)
            assert packed.offsets == cap.packed.offsets, "graph buffer layout changed"
            cap.host.numpy()[:] = packed.data
            cap.rids = tuple(e.rid for e in entries)
            cap.admissions = tuple(self.cache.admission(rid) for rid in cap.rids)
            cap.starts = np.fromiter((e.start for e in entries), np.int64, n)
        # The copy is queued, not awaited: copy and graph reach the GPU back to back.
        cap.dev.copy_(cap.host, non_blocking=True)
        if token_source is not None:
            self._take_tokens(cap.dev, cap.packed, token_source)
        if cap.copied is None:
            cap.copied = torch.cuda.Event()
        cap.copied.record()
        cap.graph.replay()
        self.graph_replays += 1
        self.steps += 1
        return cap.logits[:n]
