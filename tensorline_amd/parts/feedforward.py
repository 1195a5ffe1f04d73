"""Dense feed-forward: SwiGLU, ``down(silu(gate(h)) * up(h))``, no biases.

The reference calls the checkpoint's own module for this (tensorline/paged.py:276); the
projection names and shapes are fixed by tensorline/manager.py:52-54 and tensorline/quant.py:25.
Gate and up are fused into one [2I, H] matrix at load; SiLU is computed in float32.
"""
from __future__ import annotations

import torch

from tensorline_amd.ops import kernels
from tensorline_amd.parts.base import Linear, Part, TensorGetter, fuse_linears
from tensorline_amd.parts.registry import register_feed_forward


@register_feed_forward("swiglu")
class SwiGLU(Part):
    def __init__(self, hidden_size, prefix, dtype, device, intermediate_size: int):
        super().__init__(hidden_size, prefix, dtype, device)
        self.intermediate_size = int(intermediate_size)
        self._gate = Linear(prefix + "gate_proj", hidden_size, self.intermediate_size, False)
        self._up = Linear(prefix + "up_proj", hidden_size, self.intermediate_size, False)
        self.gate_up: Linear | None = None
        self.down = Linear(prefix + "down_proj", self.intermediate_size, hidden_size, False)

    def tensors(self):
        return {**self._gate.tensors(), **self._up.tensors(), **self.down.tensors()}

    def load(self, get: TensorGetter) -> None:
        self._gate.load(get)
        self._up.load(get)
        self.gate_up = fuse_linears(self.prefix + "gate_up_proj", [self._gate, self._up])
        self._gate.weight = self._up.weight = None
        self.down.load(get)
        self.down.prepare()

    def weight_tensors(self):
        return self.gate_up.tensors_kept() + self.down.tensors_kept()

    def library_products(self):
        return [(self.gate_up.weight, self.dtype), (self.down.weight, torch.float32)]

    @property
    def defers_norm(self) -> bool:
        return self.gate_up.shuffled is not None and self.down.shuffled is not None

    keeps_share_sums = True

    def forward(self, h, ctx, sink=None, keep_shares: bool = False):
        act = kernels.swiglu_gate_up(h, self.gate_up.weight, self.gate_up.streamed)
        return self.down(act, out_dtype=torch.float32, sink=sink, keep_shares=keep_shares)
