"""The two ends of a decoder as parts: the token embedding that starts the residual stream and
the head that turns normed rows into logits.

* **Embedding** (``@register_embedding``): ``forward(ids int32 [T]) -> float32 [T, H]``.  One that a
  head may be tied to exposes ``name`` (its tensor's checkpoint name) and ``table`` ([V, H]).
* **Head** (``@register_head``): ``load(get, embedding)``, ``optional_tensors(embedding)`` (names a
  checkpoint may hold besides the declared ones, each with the declared tensor it must equal),
  ``forward(h) -> float32 logits [R, V]`` for the wanted rows only, and ``takes_normed_rows()``:
  whether ``h`` may be :class:`tensorline_amd.ops.kernels.NormedRows` (the final norm carried by
  the head's product).

Reference: ``x = embed_tokens(ids)`` (tensorline/paged.py:240) and ``lm_head`` on the wanted rows
(paged.py:278-287); a tied head uses the embedding's table (tensorline/manager.py:65).  An
embedding scale, a bias or a cap on the logits would be other kinds registered beside these.
"""
from __future__ import annotations

import torch

from tensorline_amd.ops import kernels
from tensorline_amd.parts.base import Linear, Part, TensorGetter
from tensorline_amd.parts.registry import register_embedding, register_head
from tensorline_amd.parts.spec import TensorDecl


@register_embedding("token_embedding")
class TokenEmbedding(Part):
    def __init__(self, hidden_size, prefix, dtype, device, vocab_size: int, name: str, std: float = 0.02):
        super().__init__(hidden_size, prefix, dtype, device)
        self.vocab_size = int(vocab_size)
        self.name = prefix + name
        self.std = float(std)
        self.table: torch.Tensor | None = None

    def tensors(self):
        return {self.name: TensorDecl((self.vocab_size, self.hidden_size), "normal", self.std, "compute")}

    def load(self, get: TensorGetter) -> None:
        self.table = get(self.name)

    def weight_tensors(self):
        return [self.table]

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        return kernels.embed(ids, self.table)


@register_head("lm_head")
class LMHead(Part):
    """``logits = h W^T`` without bias, in float32.  ``tied``: W is the embedding's table (shared, not copied)."""

    def __init__(self, hidden_size, prefix, dtype, device, vocab_size: int, name: str, tied: bool = False,
                 std: float = 0.02):
        super().__init__(hidden_size, prefix, dtype, device)
        self.vocab_size = int(vocab_size)
        self.name = prefix + name
        self.tied = bool(tied)
        self.linear = Linear(self.name.removesuffix(".weight"), hidden_size, self.vocab_size, False, std)

    def tensors(self):
        return {} if self.tied else {self.name: TensorDecl((self.vocab_size, self.hidden_size), "normal", self.linear.std, "compute")}

    def optional_tensors(self, embedding) -> dict[str, str]:
        return {self.name: embedding.name} if self.tied else {}

    def load(self, get: TensorGetter, embedding=None) -> None:
        if self.tied:
            table = getattr(embedding, "table", None)
            if table is None or tuple(table.shape) != (self.vocab_size, self.hidden_size):
                raise ValueError(f"head {self.name!r} is tied, but the embedding offers no [vocab, hidden] table")
            self.linear.weight = table
        else:
            self.linear.weight = get(self.name)
        self.linear.prepare()

    def weight_tensors(self):
        return self.linear.tensors_kept()

    def takes_normed_rows(self) -> bool:
        return self.linear.shuffled is not None

    def forward(self, h) -> torch.Tensor:
        return self.linear(h, out_dtype=torch.float32)
