"""Arrangements of a layer's parts.

``prenorm`` is the residual order of the reference (tensorline/paged.py:243-247,275-276):

    x <- x + pending;  h1 = norm1(x);  x <- x + mixer(h1);  h2 = norm2(x);  pending = ffn(h2)

The feed-forward output is not added at once: it is handed to the next block (or to the final
norm) as ``pending`` and folded into that block's first fused add-and-norm.

Few-row bfloat16 steps (decoding) can do without norm kernels: when a norm is ``deferrable()`` and
the parts on both sides of it set ``defers_norm``, the product that ends the branch before the norm
adds into the residual and prepares the norm's input, and the product after it applies the
division (``tensorline_amd.ops.kernels.NormedRows``).  What is handed to the next block is then
that object instead of a pending tensor; ``next_norm`` names the norm that follows this block.
"""
from __future__ import annotations

import torch

from tensorline_amd.ops import kernels
from tensorline_amd.parts.base import Part
from tensorline_amd.parts.registry import build_part, register_block
from tensorline_amd.parts.spec import LayerSpec


@register_block("prenorm")
class PreNormBlock:
    def __init__(self, spec: LayerSpec, hidden_size: int, dtype, device):
        common = dict(hidden_size=hidden_size, dtype=dtype, device=device)
        self.spec = spec
        self.mixer_norm = build_part("norm", spec.mixer_norm, layer_prefix=spec.prefix, **common)
        self.mixer = build_part("mixer", spec.mixer, layer_prefix=spec.prefix, **common)
        self.feed_forward_norm = build_part("norm", spec.feed_forward_norm, layer_prefix=spec.prefix, **common)
        self.feed_forward = build_part("feed_forward", spec.feed_forward, layer_prefix=spec.prefix, **common)

    def parts(self) -> list[Part]:
        return [self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward]

    def takes_normed_rows(self) -> bool:
        """Whether the block before this one may hand over this block's first norm as NormedRows."""
        return _deferrable(self.mixer_norm) is not None and bool(getattr(self.mixer, "defers_norm", False))

    def forward(self, x: torch.Tensor, pending, ctx, cache, next_norm=None, pending_norm=None):
        """Updates the residual stream ``x`` in place; returns the new pending feed-forward output.
        ``pending`` is what is still to be added (a tensor, a ShareSum this block's first norm said
        it adds, or None), or the NormedRows of this block's first norm (already added).
        ``next_norm``: the norm that will take this block's output, given only when whoever applies
        it accepts NormedRows; the block may then return them.  ``pending_norm``: the norm that
        will add what this block returns, if it is one that adds a ShareSum."""
        defer = kernels.can_defer_norm(x.shape[0], self.mixer_norm.dtype)
        h = pending if isinstance(pending, kernels.NormedRows) else self.mixer_norm.forward(x, pending)
        sink = self._sink(defer, x, self.mixer, self.feed_forward_norm, self.feed_forward)
        if sink is not None:
            h = self.mixer.forward(h, ctx, cache, sink=sink)
        else:
            h = self.feed_forward_norm.forward(x, self.mixer.forward(h, ctx, cache))
        sink = self._sink(defer and next_norm is not None, x, self.feed_forward, next_norm, None)
        if sink is not None:
            return self.feed_forward.forward(h, ctx, sink=sink)
        if pending_norm is not None and getattr(self.feed_forward, "keeps_share_sums", False):
            return self.feed_forward.forward(h, ctx, keep_shares=True)
        return self.feed_forward.forward(h, ctx)

    @staticmethod
    def _sink(allowed: bool, x, producer, norm, consumer):
        """The sink for ``producer``'s last product when ``norm`` can be carried by it and by
        ``consumer`` (None: the caller vouches for the consumer)."""
        if not allowed or not getattr(producer, "defers_norm", False):
            return None
        if consumer is not None and not getattr(consumer, "defers_norm", False):
            return None
        wd = _deferrable(norm)
        return kernels.NormSink(x, wd[0], wd[1]) if wd is not None else None


def _deferrable(norm):
    fn = getattr(norm, "deferrable", None)
    return fn() if fn is not None else None
