"""Grouped-query attention over the paged cache.

One step: fused q/k/v projection (with bias), position encoding of queries and keys, write of the
new keys and values into the cache, causal attention of every token of the step over the cached
keys of its sequence, output projection (reference order: tensorline/paged.py:247-275).  All
attention, for a whole prompt, a portion of one or a single decoded token, reads the cache; the
step's own keys are in it before attention runs (paged.py:252-253).
"""
from __future__ import annotations

import torch

from tensorline_amd.ops import kernels
from tensorline_amd.parts.base import Linear, Part, TensorGetter, fuse_linears
from tensorline_amd.parts.registry import build_part, register_mixer
from tensorline_amd.parts.spec import CacheNeed, PartSpec, keys_and_values


@register_mixer("attention")
class PagedAttention(Part):
    """Parameters: head counts and size, whether q/k/v carry a bias, the position encoding, an
    optional ``window`` (a token sees only the last ``window`` keys, itself included), an optional
    ``scale`` (default head_dim^-1/2, tests/test_paged_attn.py:36), and ``kv_proj`` False for a
    layer that only reads keys and values another layer cached."""

    def __init__(self, hidden_size, prefix, dtype, device, num_heads: int, num_kv_heads: int, head_dim: int,
                 position: PartSpec, qkv_bias: bool = True, out_bias: bool = False, window: int = 0,
                 scale: float | None = None, kv_proj: bool = True):
        super().__init__(hidden_size, prefix, dtype, device)
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are not a multiple of {num_kv_heads} key/value heads")
        self.num_heads, self.num_kv_heads, self.head_dim = int(num_heads), int(num_kv_heads), int(head_dim)
        # The kernels take head sizes in steps of 16.  Another size is served at the next step: the
        # projections get rows of zeros at the end of every head when they are loaded (and the output
        # projection columns of zeros), so the added dimensions of queries, keys and values are zero,
        # add nothing to a score and come out of the weighted sum as zeros that meet zero columns.
        self.kernel_dim = -(-self.head_dim // 16) * 16
        if self.head_dim <= 0 or not kernels.attention_takes_head_dim(self.kernel_dim):
            raise ValueError(f"{prefix}: a head size of {self.head_dim} is not served: the attention kernels take "
                             "up to 256")
        self.window = int(window or 0)
        self.scale = float(scale) if scale is not None else self.head_dim ** -0.5
        self.kv_proj = bool(kv_proj)
        q_size, kv_size = self.num_heads * self.head_dim, self.num_kv_heads * self.head_dim
        self._projs = [Linear(prefix + "q_proj", hidden_size, q_size, qkv_bias)]
        if self.kv_proj:
            self._projs += [Linear(prefix + "k_proj", hidden_size, kv_size, qkv_bias),
                            Linear(prefix + "v_proj", hidden_size, kv_size, qkv_bias)]
        self.qkv: Linear | None = None
        self.o_proj = Linear(prefix + "o_proj", q_size, hidden_size, out_bias)
        self.position = build_part("position", position, head_dim=self.head_dim, device=device)

    # ---- weights -----------------------------------------------------------------------
    def tensors(self):
        out = {}
        for p in self._projs + [self.o_proj]:
            out.update(p.tensors())
        return out

    def _pad_heads(self, lin: Linear, heads: int, rows: bool) -> None:
        """Widen every head of a loaded projection from head_dim to kernel_dim with zeros: rows (and
        bias entries) of a q/k/v projection, columns of the output projection."""
        d, dp = self.head_dim, self.kernel_dim
        w = lin.weight
        if rows:
            wide = w.new_zeros(heads, dp, w.shape[1])
            wide[:, :d] = w.view(heads, d, w.shape[1])
            lin.weight, lin.out_features = wide.view(heads * dp, w.shape[1]), heads * dp
            if lin.bias is not None:
                b = lin.bias.new_zeros(heads, dp)
                b[:, :d] = lin.bias.view(heads, d)
                lin.bias = b.view(-1)
        else:
            wide = w.new_zeros(w.shape[0], heads, dp)
            wide[:, :, :d] = w.view(w.shape[0], heads, d)
            lin.weight, lin.in_features = wide.view(w.shape[0], heads * dp), heads * dp

    def load(self, get: TensorGetter) -> None:
        for p in self._projs:
            p.load(get)
        self.o_proj.load(get)
        if self.kernel_dim != self.head_dim:
            for i, p in enumerate(self._projs):
                self._pad_heads(p, self.num_heads if i == 0 else self.num_kv_heads, rows=True)
            self._pad_heads(self.o_proj, self.num_heads, rows=False)
        self.qkv = fuse_linears(self.prefix + "qkv_proj", self._projs)
        for p in self._projs:          # the fused copy is the one that is kept
            p.weight = p.bias = None
        self.o_proj.prepare()

    def weight_tensors(self):
        return self.qkv.tensors_kept() + self.o_proj.tensors_kept()

    # ---- what it keeps -------------------------------------------------------------------
    def cache_need(self) -> CacheNeed | None:
        return keys_and_values(self.num_kv_heads, self.kernel_dim, self.window)

    def state_need(self):
        return None

    # ---- one step ------------------------------------------------------------------------
    def library_products(self):
        return [(self.qkv.weight, self.dtype), (self.o_proj.weight, torch.float32)]

    @property
    def defers_norm(self) -> bool:
        return self.qkv.shuffled is not None and self.o_proj.shuffled is not None

    @staticmethod
    def step_vectors(facts) -> dict:
        """The one-token sequences of a step that also holds prompt portions, for the launch of their
        own that long contexts give them (``kernels.paged_attention``)."""
        singles = kernels.one_token_sequences(facts)
        return {"attention.single_seqs": singles} if singles else {}

    def forward(self, h, ctx, cache, sink=None):
        nkv_local = self.num_kv_heads if self.kv_proj else 0
        write = cache.write and self.kv_proj
        d = self.kernel_dim
        keys, values = cache.planes["k"], cache.planes["v"]
        qkv = None
        fused = getattr(self.position, "project_rotate_store", None)
        if fused is not None and write:
            qkv = fused(h, self.qkv, ctx.pos, self.num_heads, nkv_local, d, keys, values, cache.slots)
        if qkv is None:
            if self.qkv.bias is not None and getattr(self.position, "adds_bias", False):
                qkv = self.qkv(h, with_bias=False)           # the bias rides on the position encoding's pass
                self.position.apply_and_store(qkv, ctx.pos, self.num_heads, nkv_local, d,
                                              keys if write else None, values if write else None,
                                              cache.slots if write else None, bias=self.qkv.bias)
            else:
                qkv = self.qkv(h)
                self.position.apply_and_store(qkv, ctx.pos, self.num_heads, nkv_local, d,
                                              keys if write else None, values if write else None,
                                              cache.slots if write else None)
        o = kernels.paged_attention(qkv, keys, values, cache.tables, ctx.seq_of_token, ctx.pos,
                                    self.num_heads, self.num_kv_heads, d, self.scale,
                                    window=self.window, q_start=ctx.q_start, ctx_start=ctx.ctx_start,
                                    plan=ctx.facts, single_seqs=ctx.extra.get("attention.single_seqs"))
        return self.o_proj(o, out_dtype=torch.float32, sink=sink)
