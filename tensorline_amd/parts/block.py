"""Arrangements of a layer's parts.

``prenorm`` is the residual order of the reference (tensorline/paged.py:243-247,275-276):

    x <- x + pending;  h1 = norm1(x);  x <- x + mixer(h1);  h2 = norm2(x);  pending = ffn(h2)

The feed-forward output is not added at once: it is handed to the next block (or to the final
norm) as ``pending`` and folded into that block's first fused add-and-norm.
"""
from __future__ import annotations

import torch

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

    def forward(self, x: torch.Tensor, pending: torch.Tensor | None, ctx, cache) -> torch.Tensor:
        """Updates the residual stream ``x`` in place; returns the new pending feed-forward output."""
        h = self.mixer_norm.forward(x, pending)
        a = self.mixer.forward(h, ctx, cache)
        h = self.feed_forward_norm.forward(x, a)
        return self.feed_forward.forward(h, ctx)
