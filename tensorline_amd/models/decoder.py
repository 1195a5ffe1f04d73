"""A decoder built from a :class:`ModelSpec`: embedding, blocks in schedule order, final norm, head.

The model owns weights and the order of operations of one step; it owns no cache and no batch
logic.  ``forward(ctx, caches)`` runs exactly the tokens of ``ctx`` and returns float32 logits
for ``ctx.logit_rows`` (reference: tensorline/paged.py:240-287; the head runs on the wanted rows
only, paged.py:278-287).
"""
from __future__ import annotations

from typing import Callable

import torch

from tensorline_amd.ops import kernels
from tensorline_amd.parts.registry import BLOCKS, build_part, _ensure_builtin
from tensorline_amd.parts.spec import CacheNeed, Intake, ModelSpec, StateNeed, TensorDecl


class DecoderModel:
    def __init__(self, spec: ModelSpec, dtype: torch.dtype, device):
        _ensure_builtin()
        spec.validate()
        self.spec = spec
        self.dtype = dtype
        self.device = device
        self.hidden_size, self.vocab_size = spec.hidden_size, spec.vocab_size
        common = dict(hidden_size=spec.hidden_size, dtype=dtype, device=device)
        self.embedding = build_part("embedding", spec.embedding, layer_prefix="", vocab_size=spec.vocab_size, **common)
        self.blocks = []
        for layer in spec.layers:
            try:
                cls = BLOCKS[layer.block]
            except KeyError:
                raise ValueError(f"unknown block kind {layer.block!r}; known: {', '.join(sorted(BLOCKS))}") from None
            self.blocks.append(cls(layer, spec.hidden_size, dtype, device))
        self.schedule = spec.run_order()
        self.final_norm = build_part("norm", spec.final_norm, layer_prefix="", **common)
        self.head = build_part("head", spec.head, layer_prefix="", vocab_size=spec.vocab_size, **common)
        self._after: list[Intake | None] | None = None     # per schedule entry: what its successor takes
        self._vector_makers: list | None = None

    def _all_parts(self):
        yield self.embedding
        for b in self.blocks:
            yield from b.parts()
        yield self.final_norm
        yield self.head

    # ---- weights -----------------------------------------------------------------------
    def tensor_decls(self) -> dict[str, TensorDecl]:
        out: dict[str, TensorDecl] = {}
        for p in self._all_parts():
            out.update(p.tensors())
        return out

    def optional_tensors(self) -> dict[str, str]:
        """Names a checkpoint may also hold, with the declared tensor each must then equal."""
        fn = getattr(self.head, "optional_tensors", None)
        return fn(self.embedding) if fn is not None else {}

    def load_tensors(self, get: Callable[[str], torch.Tensor]) -> None:
        self.embedding.load(get)
        for b in self.blocks:
            for p in b.parts():
                p.load(get)
        self.final_norm.load(get)
        self.head.load(get, self.embedding)
        self._after = None

    def weight_bytes(self) -> int:
        """Bytes of weights on the device, a shared tensor counted once (reference: quant.py:107-113)."""
        seen, total = set(), 0
        for p in self._all_parts():
            for t in p.weight_tensors():
                if t is None or t.data_ptr() in seen:
                    continue
                seen.add(t.data_ptr())
                total += t.numel() * t.element_size()
        return total

    # ---- what the cache manager has to provide ------------------------------------------
    def cache_needs(self) -> list[CacheNeed | None]:
        """Per schedule entry: what its block keeps per cached token, or None."""
        return [self.blocks[e.layer].cache_need() for e in self.schedule]

    def state_needs(self) -> list[StateNeed | None]:
        """Per schedule entry: the fixed-size per-request state its block keeps, or None."""
        return [self.blocks[e.layer].state_need() for e in self.schedule]

    # ---- one step ------------------------------------------------------------------------
    def tune_library(self, rows: int) -> int:
        """Let the library choose its kernels by measurement for steps of ``rows`` tokens (a full
        prompt portion): one search per distinct product shape.  Returns how many were searched."""
        seen, done = set(), 0
        for part in self._all_parts():
            for weight, out_dtype in getattr(part, "library_products", lambda: [])():
                key = (tuple(weight.shape), weight.dtype, out_dtype)
                if key in seen:
                    continue
                seen.add(key)
                done += bool(kernels.tune_library_linear(rows, weight, out_dtype))
        return done

    def _tail_intake(self) -> Intake:
        """What the final norm and the head take from the last block."""
        carried = None
        if getattr(self.head, "takes_normed_rows", lambda: False)():
            fn = getattr(self.final_norm, "deferrable", None)
            carried = fn() if fn is not None else None
        return Intake(carried, bool(getattr(self.final_norm, "adds_share_sums", False)))

    def _negotiate(self) -> list[Intake | None]:
        """For every schedule entry the intake of whoever runs after it, or None for a block that
        takes no ``after=`` (then it returns a tensor, which everybody takes)."""
        takers = [self.blocks[e.layer] for e in self.schedule]
        intakes = [b.intake() if hasattr(b, "intake") else Intake() for b in takers[1:]] + [self._tail_intake()]
        return [nxt if hasattr(b, "intake") else None for b, nxt in zip(takers, intakes)]

    def step_vectors(self, facts) -> dict:
        """int32 index vectors that parts want on the device for a step of this shape, by name.  A
        part that has ``step_vectors(facts) -> {name: vector}`` is asked; parts of one class share
        their vectors, so one of them answers for all.  They are found in ``StepContext.extra``."""
        if self._vector_makers is None:
            seen = {}
            for p in self._all_parts():
                if hasattr(p, "step_vectors"):
                    seen.setdefault(type(p), p)
            self._vector_makers = list(seen.values())
        out: dict = {}
        for p in self._vector_makers:
            out.update(p.step_vectors(facts))
        return out

    def forward(self, ctx, caches) -> torch.Tensor:
        """``caches[i]`` is the view of the cache for schedule entry ``i``."""
        if self._after is None:
            self._after = self._negotiate()
        x = self.embedding.forward(ctx.ids)
        carry = None
        for i, e in enumerate(self.schedule):
            block, after = self.blocks[e.layer], self._after[i]
            if after is None:
                carry = block.forward(x, carry, ctx, caches[i])
            else:
                carry = block.forward(x, carry, ctx, caches[i], after=after)
        if ctx.logit_rows.numel() == 0:
            # the residual stream is complete only after the last add; nothing reads it here
            return torch.empty(0, self.vocab_size, dtype=torch.float32, device=x.device)
        if getattr(carry, "stands_for_normed_rows", False):
            # the last block's carry already is the final norm's output in the form the head takes
            # (negotiated by ``_tail_intake``); the carry knows how to give the wanted rows of itself
            h = carry if ctx.logits_for_all_rows else carry.take(ctx.logit_rows)
        else:
            h = self.final_norm.forward(x, carry, rows=ctx.logit_rows)
        return self.head.forward(h)
