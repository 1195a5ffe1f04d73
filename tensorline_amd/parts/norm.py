"""RMSNorm, fused with the residual add that precedes it.

``h = forward(x, residual)`` does ``x += residual`` on the float32 residual stream (in place)
and returns ``x / sqrt(mean(x^2) + eps) * weight`` in the activation dtype.  Sum of squares,
scaling and the residual sum are float32 (reference: tensorline/fused.py:19-32,58-69).
"""
from __future__ import annotations

import torch

from tensorline_amd.ops import kernels
from tensorline_amd.parts.base import Part, TensorGetter
from tensorline_amd.parts.registry import register_norm
from tensorline_amd.parts.spec import TensorDecl


@register_norm("rmsnorm")
class RMSNorm(Part):
    def __init__(self, hidden_size, prefix, dtype, device, eps: float, name: str = "weight"):
        super().__init__(hidden_size, prefix, dtype, device)
        self.eps = float(eps)
        self.name = prefix + name
        self.weight: torch.Tensor | None = None

    def tensors(self):
        return {self.name: TensorDecl((self.hidden_size,), "one_plus_normal", 0.1, "float32")}

    def load(self, get: TensorGetter) -> None:
        self.weight = get(self.name)

    def weight_tensors(self):
        return [self.weight]

    adds_share_sums = True

    def deferrable(self) -> tuple[torch.Tensor, float]:
        """(weight, eps): all a product needs to carry this norm (see ``Part.defers_norm``)."""
        return self.weight, self.eps

    def forward(self, x: torch.Tensor, residual=None, rows: torch.Tensor | None = None) -> torch.Tensor:
        return kernels.add_rmsnorm(x, residual, self.weight, self.eps, self.dtype, rows=rows)
