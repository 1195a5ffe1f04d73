"""From logits to tokens: greedy, temperature and top-p (reference: ``sample``,
tensorline/engine.py:42-51, and the batch arg-max of tensorline/batch_engine.py:386).

The random draw of a row is a uniform number computed from (request seed, index of the generated
token) alone, so a request's tokens do not depend on what else is in the batch.  The reference
uses torch's global generator instead; a per-request seed is this engine's addition.
"""
from __future__ import annotations

import torch

from tensorline_amd.ops import kernels

_MASK64 = (1 << 64) - 1


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK64
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK64
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _MASK64
    return x ^ (x >> 31)


def uniform_for(seed: int, index: int) -> float:
    """A number in [0, 1) with 24 random bits, a pure function of (seed, index)."""
    h = _splitmix64(_splitmix64(seed & _MASK64) ^ (index & _MASK64))
    return (h >> 40) / float(1 << 24)


class Sampler:
    def __init__(self, device):
        self.device = device

    def sample_device(self, logits: torch.Tensor, temperatures: list[float], top_ps: list[float],
                      seeds: list[int], indices: list[int]) -> torch.Tensor:
        """One token per row of float32 ``logits`` [R, V], as an int32 tensor on the device: nothing
        is awaited, so the caller may queue more work before it looks at the tokens."""
        R = logits.shape[0]
        if R == 0:
            return torch.empty(0, dtype=torch.int32, device=logits.device)
        if all(t <= 0 for t in temperatures):
            return kernels.argmax(logits)
        u = [uniform_for(s, i) for s, i in zip(seeds, indices)]
        params = torch.tensor([temperatures, top_ps, u], dtype=torch.float32).to(self.device)
        return kernels.sample(logits, params[0], params[1], params[2],
                              any_top_p=any(p < 1.0 for p in top_ps),
                              any_greedy=any(t <= 0 for t in temperatures))

    def sample(self, logits: torch.Tensor, temperatures: list[float], top_ps: list[float],
               seeds: list[int], indices: list[int]) -> list[int]:
        """The same, awaited and as a list."""
        return self.sample_device(logits, temperatures, top_ps, seeds, indices).tolist()
