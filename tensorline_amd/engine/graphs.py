"""HIP-graph replay of pure decode steps.

A decode step at small batch is a few hundred short kernels; launching them one by one costs more
than running them.  A graph records the whole step once and replays it with one launch
(reference: ``CudaGraphDecoder``, tensorline/cuda_graphs.py:38-126).  Graphs need fixed shapes and
addresses, so:

* the batch is padded to a bucket (1, 2, 4, ... max_num_seqs); one graph per bucket, captured at
  first use or ahead of time by ``warmup``;
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

import torch

from tensorline_amd.cache.manager import CacheManager
from tensorline_amd.engine.batch import StepEntry
from tensorline_amd.engine.runner import ModelRunner


def _pow2_upto(limit: int) -> list[int]:
    out, b = [], 1
    while b < limit:
        out.append(b)
        b *= 2
    return out + [limit]


class _Captured:
    def __init__(self, graph, dev, host, logits, packed):
        self.graph, self.dev, self.host, self.logits, self.packed = graph, dev, host, logits, packed


class GraphRunner(ModelRunner):
    def __init__(self, model, cache: CacheManager, max_batch: int, max_blocks_per_seq: int):
        super().__init__(model, cache)
        self.batch_buckets = _pow2_upto(max_batch)
        self.max_blocks = max_blocks_per_seq
        self.graphs: dict[int, _Captured] = {}
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
                            scratch_slot=cache.scratch_slot)
        return packed

    @torch.inference_mode()
    def _capture(self, B: int) -> _Captured:
        packed = self._padding_batch(B)
        packed.plan.max_context = self.max_blocks * self.cache.page_size
        packed.plan.decode_only = True
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
        self.graphs[B] = cap
        return cap

    def warmup(self, max_context_tokens: int = 0) -> int:
        """Capture every batch bucket before serving, largest first, so that no request pays for a
        capture (tensorline/cuda_graphs.py:84-96).  Captures touch only the scratch page."""
        for B in reversed(self.batch_buckets):
            if B not in self.graphs:
                self._capture(B)
        torch.cuda.synchronize()
        return len(self.graphs)

    # ---- one step ------------------------------------------------------------------------------
    @torch.inference_mode()
    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        if not self.can_run(entries):
            return super().step(entries)
        n = len(entries)
        B = self._bucket(n)
        cap = self.graphs.get(B) or self._capture(B)
        ng = len(self.cache.groups)
        packed = self.pack(entries, pad_seqs=B, pad_nb=[self.max_blocks] * ng)
        assert packed.offsets == cap.packed.offsets, "graph buffer layout changed"
        cap.host.numpy()[:] = packed.data
        cap.dev.copy_(cap.host, non_blocking=False)
        cap.graph.replay()
        self.graph_replays += 1
        self.steps += 1
        return cap.logits[:n]
