"""What every part has in common: it declares the checkpoint tensors it needs and takes them.

A part is built from sizes and constants only (its ``PartSpec.params``) plus ``hidden_size``,
the checkpoint ``prefix`` it lives under, the compute ``dtype`` and the ``device``.  It does not
know which model it is in.
"""
from __future__ import annotations

from typing import Callable

import torch

from tensorline_amd.ops import kernels
from tensorline_amd.parts.spec import TensorDecl

TensorGetter = Callable[[str], torch.Tensor]


class Part:
    def __init__(self, hidden_size: int, prefix: str, dtype: torch.dtype, device):
        self.hidden_size = int(hidden_size)
        self.prefix = prefix
        self.dtype = dtype
        self.device = device

    def tensors(self) -> dict[str, TensorDecl]:
        """Checkpoint name -> declaration, for every tensor this part reads."""
        return {}

    def load(self, get: TensorGetter) -> None:
        """Take the declared tensors; ``get(name)`` returns one on the device in its storage dtype."""

    def weight_tensors(self) -> list[torch.Tensor]:
        """Device tensors this part keeps (for byte accounting)."""
        return []

    def library_products(self) -> list[tuple[torch.Tensor, torch.dtype]]:
        """(weight, output dtype) of the products this part hands to the library in many-row steps."""
        return []

    # Optional hand-off of the norms to the products around them (few-row bfloat16 steps).  A mixer
    # or feed-forward that sets ``defers_norm`` takes :class:`tensorline_amd.ops.kernels.NormedRows`
    # as its input and a ``sink`` (:class:`tensorline_amd.ops.kernels.NormSink`) keyword: with a sink
    # its last product adds into the residual and returns the next norm's NormedRows instead of its
    # own output.  A norm that can be handed off this way returns (weight, eps) from ``deferrable()``.
    # Parts without these never see either object.
    defers_norm = False

    # Optional hand-off of a product's K shares to the norm that adds it to the residual (many-row
    # bfloat16 steps).  A feed-forward that sets ``keeps_share_sums`` takes a ``keep_shares`` keyword
    # and may then return :class:`tensorline_amd.ops.kernels.ShareSum` instead of a tensor; a norm
    # that sets ``adds_share_sums`` takes one as its residual.  The block asks only when both do.
    keeps_share_sums = False
    adds_share_sums = False


class Linear:
    """``y = x W^T + b`` with W [out, in] as checkpoints store it (reference: tensorline/quant.py:3)."""

    def __init__(self, name: str, in_features: int, out_features: int, bias: bool, std: float = 0.02):
        self.name = name
        self.in_features, self.out_features, self.has_bias, self.std = in_features, out_features, bias, std
        self.weight: torch.Tensor | None = None
        self.bias: torch.Tensor | None = None
        self.shuffled: torch.Tensor | None = None     # the copy few-row bfloat16 products stream
        self.shuffled_float: torch.Tensor | None = None   # the same for a float32 weight (the 32-bit path's decode steps)

    def tensors(self) -> dict[str, TensorDecl]:
        out = {self.name + ".weight": TensorDecl((self.out_features, self.in_features), "normal", self.std, "compute")}
        if self.has_bias:
            out[self.name + ".bias"] = TensorDecl((self.out_features,), "normal", self.std, "float32")
        return out

    def load(self, get: TensorGetter) -> None:
        self.weight = get(self.name + ".weight")
        self.bias = get(self.name + ".bias") if self.has_bias else None

    def prepare(self) -> "Linear":
        """Make the second, matrix-core ordered copy of a bfloat16 weight.  Decode steps stream
        that copy, many-row steps hand the row-major one to the library: twice the bytes, for
        which 288 GB of HBM has room."""
        self.shuffled = kernels.shuffle_weight(self.weight)
        self.shuffled_float = kernels.shuffle_weight_float(self.weight)
        return self

    def tensors_kept(self) -> list[torch.Tensor]:
        return [t for t in (self.weight, self.bias, self.shuffled, self.shuffled_float) if t is not None]

    @property
    def streamed(self) -> torch.Tensor | None:
        """The matrix-core ordered copy few-row products stream, of whichever type the weight has."""
        return self.shuffled if self.shuffled is not None else self.shuffled_float

    def __call__(self, x, out_dtype: torch.dtype | None = None, sink=None, with_bias: bool = True,
                 keep_shares: bool = False):
        return kernels.linear(x, self.weight, self.bias if with_bias else None, out_dtype=out_dtype,
                              shuffled=self.streamed, sink=sink, keep_shares=keep_shares)


def fuse_linears(name: str, parts: list[Linear]) -> Linear:
    """One Linear whose rows are the rows of ``parts`` in order: one matrix product instead of
    several over the same input."""
    fused = Linear(name, parts[0].in_features, sum(p.out_features for p in parts), any(p.has_bias for p in parts))
    fused.weight = torch.cat([p.weight for p in parts], dim=0).contiguous()
    if fused.has_bias:
        fused.bias = torch.cat([
            p.bias if p.bias is not None else torch.zeros(p.out_features, dtype=torch.float32, device=p.weight.device)
            for p in parts]).contiguous()
    return fused.prepare()
