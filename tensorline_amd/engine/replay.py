"""Trace replay: feed given token ids through the model step by step and write logits.

Nothing is sampled.  A trace is a stream of JSON lines, one step each::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

All entries of a step run as one batch through :class:`tensorline_amd.engine.runner.ModelRunner`,
the step function generation uses, over pages from the same cache manager.  For a step that wants
logits, ``<out>/<step>.f32`` holds them as little-endian float32 [wanted, vocab], in the order of
the entries and of their ``want`` lists.  After every step a line ``done <step>`` is printed.
Requests named in ``end`` give their pages back after the step.

Nearest things in the reference: driving ``PagedModel.forward`` with hand-made chunks and tables
(tests/test_batching.py:54-64, tests/test_cuda_graphs.py:23-44).
"""
from __future__ import annotations

import argparse
import json
import os
import sys

import numpy as np
import torch

from tensorline_amd.cache.manager import CacheManager
from tensorline_amd.engine.batch import StepEntry
from tensorline_amd.engine.runner import ModelRunner

ROUND_TOKENS = 64       # a request's token count is rounded up to this when the pool is sized


class TraceError(RuntimeError):
    pass


class TraceSession:
    """Live requests of a trace and the cache they share."""

    def __init__(self, model, max_tokens: int, page_size: int = 16, max_requests: int = 8, graphs: bool = False):
        """``max_tokens``: the most tokens live requests hold at any time (each request's count
        rounded up to 64); ``max_requests``: the most requests live at a time.  ``graphs``: steps
        that are pure decoding replay a HIP graph, as the engine's do, instead of running eagerly."""
        if ROUND_TOKENS % page_size:
            raise ValueError(f"page size {page_size} must divide {ROUND_TOKENS}")
        if max_requests <= 0:
            raise ValueError("max_requests must be positive")
        num_blocks = max(1, -(-int(max_tokens) // page_size))
        self.model = model
        self.cache = CacheManager(model.cache_needs(), model.schedule, model.state_needs(), page_size=page_size,
                                  num_blocks=num_blocks, max_requests=max_requests, dtype=model.dtype,
                                  device=model.device, prefix_caching=False)
        if graphs:
            from tensorline_amd.engine.graphs import GraphRunner
            # one request can hold the whole pool at most: that bounds every page table
            self.runner = GraphRunner(model, self.cache, max_batch=max_requests, max_blocks_per_seq=num_blocks)
        else:
            self.runner = ModelRunner(model, self.cache)
        self.computed: dict[str, int] = {}

    def step(self, entries: list[dict], end: list[str] | tuple = ()) -> np.ndarray | None:
        """Run one step; returns the wanted logits [wanted, vocab] as float32, or None."""
        batch: list[StepEntry] = []
        seen = set()
        for e in entries:
            rid = str(e["id"])
            if rid in seen:
                raise TraceError(f"request {rid!r} appears twice in one step")
            seen.add(rid)
            tokens = [int(t) for t in e["tokens"]]
            if not tokens:
                raise TraceError(f"request {rid!r} brings no tokens")
            vocab = getattr(self.model, "vocab_size", None)
            if vocab is not None and any(t < 0 or t >= vocab for t in tokens):
                raise TraceError(f"request {rid!r} brings a token id outside [0, {vocab})")
            if rid not in self.computed:
                if self.cache.add_request(rid) is None:
                    raise TraceError(f"more than {self.cache.max_requests} requests are live at once (--max-requests)")
                self.computed[rid] = 0
            start = self.computed[rid]
            if not self.cache.grow(rid, start + len(tokens)):
                raise TraceError(
                    f"out of cache pages at request {rid!r}: the pool holds {self.cache.num_blocks} pages of "
                    f"{self.cache.page_size} tokens (--max-tokens), {self.cache.min_free()} are free")
            batch.append(StepEntry(rid, tokens, start, [int(w) for w in e.get("want", [])]))
        logits = None
        if batch:
            out = self.runner.step(batch)
            for b in batch:
                self.computed[b.rid] += len(b.tokens)
                self.cache.trim(b.rid, self.computed[b.rid])
            if out.shape[0]:
                logits = out.to(torch.float32).cpu().numpy()     # a copy: a replayed graph writes its logits in place
        for rid in end:
            rid = str(rid)
            if rid in self.computed:
                self.cache.release(rid)
                del self.computed[rid]
        return logits


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser("trace_run", description="replay a token trace through the engine and write logits")
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64); sizes the cache")
    ap.add_argument("--block-size", type=int, default=16, help="tokens per cache page")
    ap.add_argument("--max-requests", type=int, default=8, help="most requests live at any time")
    ap.add_argument("--graphs", action="store_true", help="replay HIP graphs for steps that only decode, as serving does")
    ap.add_argument("--device", default="cuda:0")
    return ap


def main(argv=None, stdin=None, stdout=None) -> int:
    args = build_parser().parse_args(argv)
    stdin = stdin or sys.stdin
    stdout = stdout or sys.stdout
    from tensorline_amd.engine.loading import load_model
    from tensorline_amd.ops import kernels

    kernels.require_gpu(args.device)
    os.makedirs(args.out, exist_ok=True)
    model, _ = load_model(args.model, args.dtype, args.device)
    session = TraceSession(model, args.max_tokens, page_size=args.block_size, max_requests=args.max_requests,
                           graphs=args.graphs)
    for line in stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        logits = session.step(rec.get("entries", []), rec.get("end", []))
        if logits is not None:
            logits.astype("<f4").tofile(os.path.join(args.out, f"{step}.f32"))
        print(f"done {step}", file=stdout, flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
