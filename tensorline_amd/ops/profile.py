"""Time of one step by class of kernel, measured with HIP events around every launch.

The reference reports such a breakdown by hand (README.md:80-86,248-259: time inside the graph,
fused norm and RoPE, sampling).  Here ``KernelTimer`` wraps the one function through which every
own kernel is launched (``kernels._call``) and the one through which many-row products go to the
library (``kernels._library_linear``); each call is bracketed by two events on the current stream
and booked to a class by its entry point's name:

    products    tl_gemm_*, library products
    attention   tl_attention_*
    norm_rope   tl_add_rmsnorm, tl_rope_store, tl_embed, tl_silu_mul (the passes over activations)
    sampling    tl_argmax*, tl_sample

The step has to run eagerly (a replayed graph is one launch); events between the kernels cost a
few microseconds each, so the classes' sum is an upper bound of the graph's time, and ``host_ms``
(the time the host needs to issue the step, nothing awaited) tells what a graph saves.
"""
from __future__ import annotations

import time
from contextlib import contextmanager

import torch

from tensorline_amd.ops import kernels

CLASSES = ("products", "attention", "norm_rope", "sampling")


def kernel_class(entry_point: str) -> str:
    if entry_point.startswith("tl_gemm"):
        return "products"
    if entry_point.startswith("tl_attention"):
        return "attention"
    if entry_point.startswith(("tl_argmax", "tl_sample")):
        return "sampling"
    return "norm_rope"


class KernelTimer:
    def __init__(self):
        self._spans: list[tuple[str, str, torch.cuda.Event, torch.cuda.Event]] = []
        self.host_ms = 0.0

    @contextmanager
    def measuring(self):
        """Inside: every kernel launch is bracketed by events.  On leaving, the device is awaited."""
        call, library = kernels._call, kernels._library_linear

        def timed_call(name, *args):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            try:
                return call(name, *args)
            finally:
                e1.record()
                self._spans.append((kernel_class(name), name, e0, e1))

        def timed_library(*args, **kw):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            try:
                return library(*args, **kw)
            finally:
                e1.record()
                self._spans.append(("products", "library product", e0, e1))

        kernels._call, kernels._library_linear = timed_call, timed_library
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        try:
            yield self
            self.host_ms += (time.perf_counter() - t0) * 1e3
            torch.cuda.synchronize()
        finally:
            kernels._call, kernels._library_linear = call, library

    def summary(self) -> dict:
        """Milliseconds and launches per class, and the longest entry points."""
        ms = {c: 0.0 for c in CLASSES}
        launches = {c: 0 for c in CLASSES}
        by_name: dict[str, float] = {}
        for cls, name, e0, e1 in self._spans:
            t = e0.elapsed_time(e1)
            ms[cls] += t
            launches[cls] += 1
            by_name[name] = by_name.get(name, 0.0) + t
        top = sorted(by_name.items(), key=lambda kv: -kv[1])[:6]
        return {"ms": {c: round(v, 4) for c, v in ms.items()}, "launches": launches,
                "kernels_ms": round(sum(ms.values()), 4), "host_ms": round(self.host_ms, 4),
                "top": {n: round(v, 4) for n, v in top}}
