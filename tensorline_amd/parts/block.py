"""Arrangements of a layer's parts.

What a model asks of a block (any class registered with ``@register_block``, built as
``cls(layer_spec, hidden_size, dtype, device)``):

* ``parts()``: the parts it is made of (for tensor declarations, loading, byte counts);
* ``cache_need()`` / ``state_need()``: what its mixer keeps per token and per request, or None;
* ``forward(x, carry, ctx, cache) -> carry``: updates the float32 residual stream ``x`` in place.
  ``carry`` is what the block before left to be added (a tensor, or None for the first block);
  what it returns is what is left for whoever runs next to add.
* optionally ``intake() -> Intake``: what else it can take as ``carry`` in place of a tensor.  A
  block that has it is also called with ``after=``, the intake of whoever runs next, and may
  return a carry in one of the forms that intake allows.  A block without it is only ever handed
  plain tensors and its successor only ever gets one from it.

``prenorm`` is the residual order of the reference (tensorline/paged.py:243-247,275-276):

    x <- x + carry;  h1 = norm1(x);  x <- x + mixer(h1);  h2 = norm2(x);  carry = ffn(h2)

The feed-forward output is not added at once: it is folded into the next block's (or the final
norm's) fused add-and-norm.

Few-row bfloat16 steps (decoding) can do without norm kernels: when a norm is ``deferrable()`` and
the parts on both sides of it set ``defers_norm``, the product that ends the branch before the norm
adds into the residual and prepares the norm's input, and the product after it applies the
division (``tensorline_amd.ops.kernels.NormedRows``).  The carry is then that object; the intake
says for which norm the successor takes it.
"""
from __future__ import annotations

import torch

from tensorline_amd.ops import kernels
from tensorline_amd.parts.base import Part
from tensorline_amd.parts.registry import build_part, register_block
from tensorline_amd.parts.spec import Intake, LayerSpec


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

    def cache_need(self):
        fn = getattr(self.mixer, "cache_need", None)
        return fn() if fn is not None else None

    def state_need(self):
        fn = getattr(self.mixer, "state_need", None)
        return fn() if fn is not None else None

    def intake(self) -> Intake:
        """This block's first norm as NormedRows, if that norm can be carried and the mixer applies
        it; a ShareSum, if that norm adds one."""
        carried = _deferrable(self.mixer_norm) if getattr(self.mixer, "defers_norm", False) else None
        return Intake(carried, bool(getattr(self.mixer_norm, "adds_share_sums", False)))

    def forward(self, x: torch.Tensor, carry, ctx, cache, after: Intake | None = None):
        """``carry``: a tensor or None, or one of the forms this block's ``intake()`` offers: a
        ShareSum for its first norm to add, or that norm's NormedRows (already added to ``x``).
        ``after``: the intake of whoever runs next."""
        after = after or Intake()
        defer = kernels.can_defer_norm(x.shape[0], self.mixer_norm.dtype)
        h = carry if isinstance(carry, kernels.NormedRows) else self.mixer_norm.forward(x, carry)
        sink = self._sink(defer, x, self.mixer, _deferrable(self.feed_forward_norm), self.feed_forward)
        if sink is not None:
            h = self.mixer.forward(h, ctx, cache, sink=sink)
        else:
            h = self.feed_forward_norm.forward(x, self.mixer.forward(h, ctx, cache))
        sink = self._sink(defer, x, self.feed_forward, after.normed_rows_for, None)
        if sink is not None:
            return self.feed_forward.forward(h, ctx, sink=sink)
        if after.share_sums and getattr(self.feed_forward, "keeps_share_sums", False):
            return self.feed_forward.forward(h, ctx, keep_shares=True)
        return self.feed_forward.forward(h, ctx)

    @staticmethod
    def _sink(allowed: bool, x, producer, carried_norm, consumer):
        """The sink for ``producer``'s last product when the norm after it (``carried_norm`` =
        (weight, eps), None: it cannot be carried) can ride on it and on ``consumer`` (None: whoever
        offered the norm vouches for the consumer)."""
        if not allowed or carried_norm is None or not getattr(producer, "defers_norm", False):
            return None
        if consumer is not None and not getattr(consumer, "defers_norm", False):
            return None
        return kernels.NormSink(x, carried_norm[0], carried_norm[1])


def _deferrable(norm):
    fn = getattr(norm, "deferrable", None)
    return fn() if fn is not None else None
