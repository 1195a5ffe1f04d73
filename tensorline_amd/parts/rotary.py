"""Position encodings.  A position encoding owns two things: what is done to the query and key
heads of a step's tokens given their positions, and the write of keys and values into the paged
cache (fused, because the rotated key is what the cache holds; reference: paged.py:251-253).

Interface: ``apply_and_store(qkv, pos, num_heads, num_kv_heads, head_dim, k_cache, v_cache,
slots)`` rotates the query heads of the fused projection in place and stores keys and values at
``slots`` (``k_cache`` None: nothing is stored).  One that sets ``adds_bias`` also takes
``bias=``, the projection's bias still to be added (the mixer then leaves it out of the product:
one pass over the activations less).  A position encoding may also offer
``project_rotate_store(h, qkv_linear, ...)``, which does the projection as well and returns the
queries, or None to decline; the attention mixer tries it first.
"""
from __future__ import annotations

import torch

from tensorline_amd.ops import kernels
from tensorline_amd.parts.registry import register_position


@register_position("rope")
class RotaryEmbedding:
    """Rotate-half RoPE over the first ``rotary_dim`` dims of a head:
    theta_i = pos * base^(-2i / rotary_dim), angles in float32 (reference: fused.py:34-51; the
    table layout cat(cos, cos) is pinned by tests/test_quant.py:116-118)."""

    def __init__(self, head_dim: int, device, theta: float, rotary_dim: int | None = None):
        self.head_dim = int(head_dim)
        self.theta = float(theta)
        self.rotary_dim = int(rotary_dim) if rotary_dim is not None else self.head_dim
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and within the head size {self.head_dim}")
        # The exponent and the power are evaluated in float64 and rounded once to float32.
        idx = torch.arange(0, self.rotary_dim, 2, dtype=torch.float64)
        inv = torch.pow(torch.tensor(self.theta, dtype=torch.float64), -idx / self.rotary_dim)
        self.inv_freq = inv.to(torch.float32).to(device)

    adds_bias = True     # apply_and_store takes the projection's bias and adds it on the way

    def apply_and_store(self, qkv, pos, num_heads, num_kv_heads, head_dim, k_cache, v_cache, slots, bias=None) -> None:
        kernels.rope_store(qkv, pos, self.inv_freq, num_heads, num_kv_heads, head_dim, k_cache, v_cache, slots, bias)

    def project_rotate_store(self, h, qkv_linear, pos, num_heads, num_kv_heads, head_dim, k_cache, v_cache, slots):
        """Optional shortcut for few-row steps: projection, rotation and cache write in one kernel.
        Returns the rotated queries [T, nq*d], or None when that kernel does not take the case."""
        if self.rotary_dim != head_dim or k_cache is None:
            return None
        return kernels.qkv_rope_store(h, qkv_linear.shuffled, qkv_linear.bias, pos, self.inv_freq, num_heads,
                                      num_kv_heads, head_dim, k_cache, v_cache, slots)


@register_position("none")
class NoPosition:
    """No position encoding: keys and values are stored as they are."""

    def __init__(self, head_dim: int, device):
        self.head_dim = int(head_dim)

    adds_bias = True

    def apply_and_store(self, qkv, pos, num_heads, num_kv_heads, head_dim, k_cache, v_cache, slots, bias=None) -> None:
        if k_cache is not None or bias is not None:
            kernels.rope_store(qkv, pos, None, num_heads, num_kv_heads, head_dim, k_cache, v_cache, slots, bias)
