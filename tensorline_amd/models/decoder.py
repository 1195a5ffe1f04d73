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
from tensorline_amd.parts.base import Linear
from tensorline_amd.parts.registry import BLOCKS, build_part, _ensure_builtin
from tensorline_amd.parts.spec import CacheNeed, ModelSpec, StateNeed, TensorDecl


class DecoderModel:
    def __init__(self, spec: ModelSpec, dtype: torch.dtype, device):
        _ensure_builtin()
        spec.validate()
        self.spec = spec
        self.dtype = dtype
        self.device = device
        self.hidden_size, self.vocab_size = spec.hidden_size, spec.vocab_size
        self.blocks = []
        for layer in spec.layers:
            try:
                cls = BLOCKS[layer.block]
            except KeyError:
                raise ValueError(f"unknown block kind {layer.block!r}; known: {', '.join(sorted(BLOCKS))}") from None
            self.blocks.append(cls(layer, spec.hidden_size, dtype, device))
        self.schedule = spec.run_order()
        self.final_norm = build_part("norm", spec.final_norm, layer_prefix="", hidden_size=spec.hidden_size,
                                     dtype=dtype, device=device)
        self.embed_name = spec.embedding.params["name"]
        self.head_name = spec.head.params["name"]
        self.tied = bool(spec.head.params.get("tied", False))
        self.embed_table: torch.Tensor | None = None
        self.head = Linear(self.head_name.removesuffix(".weight"), spec.hidden_size, spec.vocab_size, False)

    # ---- weights -----------------------------------------------------------------------
    def tensor_decls(self) -> dict[str, TensorDecl]:
        H, V = self.hidden_size, self.vocab_size
        out: dict[str, TensorDecl] = {self.embed_name: TensorDecl((V, H), "normal", 0.02, "compute")}
        for b in self.blocks:
            for p in b.parts():
                out.update(p.tensors())
        out.update(self.final_norm.tensors())
        if not self.tied:
            out[self.head_name] = TensorDecl((V, H), "normal", 0.02, "compute")
        return out

    def optional_tensors(self) -> dict[str, str]:
        """Names a checkpoint may also hold, with the declared tensor each must then equal."""
        return {self.head_name: self.embed_name} if self.tied else {}

    def load_tensors(self, get: Callable[[str], torch.Tensor]) -> None:
        self.embed_table = get(self.embed_name)
        for b in self.blocks:
            for p in b.parts():
                p.load(get)
        self.final_norm.load(get)
        self.head.weight = self.embed_table if self.tied else get(self.head_name)
        self.head.prepare()

    def weight_bytes(self) -> int:
        """Bytes of weights on the device, a shared tensor counted once (reference: quant.py:107-113)."""
        seen, total = set(), 0
        tensors = [self.embed_table] + self.head.tensors_kept() + self.final_norm.weight_tensors()
        for b in self.blocks:
            for p in b.parts():
                tensors += p.weight_tensors()
        for t in tensors:
            if t is None or t.data_ptr() in seen:
                continue
            seen.add(t.data_ptr())
            total += t.numel() * t.element_size()
        return total

    # ---- what the cache manager has to provide ------------------------------------------
    def cache_needs(self) -> list[CacheNeed | None]:
        """Per schedule entry: the keys/values its mixer keeps per token, or None."""
        out = []
        for e in self.schedule:
            mixer = self.blocks[e.layer].mixer
            need = mixer.cache_need() if hasattr(mixer, "cache_need") else None
            out.append(need)
        return out

    def state_needs(self) -> list[StateNeed | None]:
        """Per schedule entry: the fixed-size per-request state its mixer keeps, or None."""
        out = []
        for e in self.schedule:
            mixer = self.blocks[e.layer].mixer
            out.append(mixer.state_need() if hasattr(mixer, "state_need") else None)
        return out

    # ---- one step ------------------------------------------------------------------------
    def tune_library(self, rows: int) -> int:
        """Let the library choose its kernels by measurement for steps of ``rows`` tokens (a full
        prompt portion): one search per distinct product shape.  Returns how many were searched."""
        seen, done = set(), 0
        for block in self.blocks:
            for part in block.parts():
                for weight, out_dtype in getattr(part, "library_products", lambda: [])():
                    key = (tuple(weight.shape), weight.dtype, out_dtype)
                    if key in seen:
                        continue
                    seen.add(key)
                    done += bool(kernels.tune_library_linear(rows, weight, out_dtype))
        return done

    def forward(self, ctx, caches) -> torch.Tensor:
        """``caches[i]`` is the view of the cache for schedule entry ``i``."""
        x = kernels.embed(ctx.ids, self.embed_table)
        pending = None
        last = len(self.schedule) - 1
        for i, e in enumerate(self.schedule):
            block = self.blocks[e.layer]
            if getattr(block, "takes_normed_rows", None) is None:
                pending = block.forward(x, pending, ctx, caches[i])      # a block that knows no hand-off
                continue
            # the norm after this block: as next_norm if whoever applies it can take it as
            # NormedRows, as pending_norm if it adds a product left in its K shares
            next_norm = after = None
            if i < last:
                nxt = self.blocks[self.schedule[i + 1].layer]
                after = getattr(nxt, "mixer_norm", None)
                if getattr(nxt, "takes_normed_rows", lambda: False)():
                    next_norm = nxt.mixer_norm
            else:
                after = self.final_norm
                if self.head.shuffled is not None:
                    next_norm = self.final_norm
            pending_norm = after if getattr(after, "adds_share_sums", False) else None
            pending = block.forward(x, pending, ctx, caches[i], next_norm=next_norm, pending_norm=pending_norm)
        if ctx.logit_rows.numel() == 0:
            # the residual stream is complete only after the last add; nothing reads it here
            return torch.empty(0, self.vocab_size, dtype=torch.float32, device=x.device)
        if isinstance(pending, kernels.NormedRows):
            h = pending if ctx.logits_for_all_rows else pending.take(ctx.logit_rows)
        else:
            h = self.final_norm.forward(x, pending, rows=ctx.logit_rows)
        return self.head(h, out_dtype=torch.float32)
