"""Data that describes a model: which parts each layer is made of and in which order layers run.

A model is a :class:`ModelSpec`.  Each layer names its parts by *kind* with their sizes and
constants as parameters (:class:`PartSpec`); the kinds are looked up in the registries of
:mod:`tensorline_amd.parts.registry`.  Different layers may use different mixers and
feed-forwards.  The order of execution is data too: ``schedule`` lists layer indices, may name a
layer twice (its weights run twice, each run with a cache of its own), and an entry may read the
cache another entry wrote instead of writing one itself.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping


@dataclass(frozen=True)
class PartSpec:
    """``kind`` picks the class; ``params`` are its sizes and constants; ``prefix`` is where its
    tensors live below the layer's checkpoint prefix (e.g. ``"self_attn."``)."""
    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)
    prefix: str = ""

    def with_params(self, **kw) -> "PartSpec":
        return PartSpec(self.kind, {**self.params, **kw}, self.prefix)


@dataclass(frozen=True)
class TensorDecl:
    """A tensor a part expects in the checkpoint.

    ``storage`` says how it is kept on the device: ``"compute"`` in the engine's dtype
    (bfloat16 or float32), ``"float32"`` always in 32-bit (norm weights, biases and anything a
    checkpoint stores in 32-bit on purpose), ``"int32"`` for integer tables.
    ``init``/``std`` drive the random-weights mode: ``"normal"`` is N(0, std), ``"one_plus_normal"``
    is 1 + N(0, std)."""
    shape: tuple[int, ...]
    init: str = "normal"
    std: float = 0.02
    storage: str = "compute"


@dataclass(frozen=True)
class LayerSpec:
    prefix: str                       # checkpoint prefix of the layer, e.g. "model.layers.3."
    mixer: PartSpec
    feed_forward: PartSpec
    mixer_norm: PartSpec
    feed_forward_norm: PartSpec
    block: str = "prenorm"            # the arrangement of the four parts


@dataclass(frozen=True)
class ScheduleEntry:
    layer: int                        # index into ModelSpec.layers
    cache_from: int | None = None     # index of the schedule entry whose cache this run reads


@dataclass(frozen=True)
class Intake:
    """What whoever runs after a block can take in place of a plain pending tensor; a block is
    told the intake of its successor and may answer with the cheaper form.
    ``normed_rows_for``: (weight, eps) of the norm the successor applies first, if it takes that
    norm's input as ``tensorline_amd.ops.kernels.NormedRows``.  ``share_sums``: its first norm adds a
    product left in its shares of K (``tensorline_amd.ops.kernels.ShareSum``)."""
    normed_rows_for: tuple | None = None
    share_sums: bool = False


@dataclass(frozen=True)
class ModelSpec:
    hidden_size: int
    vocab_size: int
    embedding: PartSpec
    layers: tuple[LayerSpec, ...]
    final_norm: PartSpec
    head: PartSpec
    schedule: tuple[ScheduleEntry, ...] = ()
    max_position: int = 1 << 30
    eos_token_ids: tuple[int, ...] = ()

    def run_order(self) -> tuple[ScheduleEntry, ...]:
        return self.schedule or tuple(ScheduleEntry(i) for i in range(len(self.layers)))

    def validate(self) -> None:
        order = self.run_order()
        for n, e in enumerate(order):
            if not 0 <= e.layer < len(self.layers):
                raise ValueError(f"schedule entry {n} names layer {e.layer}; the model has {len(self.layers)}")
            if e.cache_from is not None:
                if not 0 <= e.cache_from < n:
                    raise ValueError(f"schedule entry {n} reads the cache of entry {e.cache_from}, "
                                     "which does not run before it")
                if order[e.cache_from].cache_from is not None:
                    raise ValueError(f"schedule entry {n} reads the cache of entry {e.cache_from}, "
                                     "which has no cache of its own")


@dataclass(frozen=True)
class CachePlane:
    """One tensor a mixer keeps for every cached token: ``shape`` per token, in the cache's dtype
    (``dtype`` "compute") or a fixed one.  The cache manager lays it out in pages and knows nothing
    else about it: ``token_axis`` "first" gives storage ``[pages, page, *shape]`` (a token's values
    contiguous), "last" gives ``[pages, *shape, page]`` (a page's tokens contiguous innermost)."""
    name: str
    shape: tuple[int, ...]
    token_axis: str = "first"
    dtype: str = "compute"

    def __post_init__(self):
        if self.token_axis not in ("first", "last"):
            raise ValueError(f"cache plane {self.name!r}: token_axis must be 'first' or 'last'")
        if not self.shape or min(self.shape) <= 0:
            raise ValueError(f"cache plane {self.name!r}: a token's shape must be non-empty and positive")

    def storage_shape(self, pages: int, page_size: int) -> tuple[int, ...]:
        return (pages, page_size, *self.shape) if self.token_axis == "first" else (pages, *self.shape, page_size)

    def values_per_token(self) -> int:
        n = 1
        for d in self.shape:
            n *= d
        return n


@dataclass(frozen=True)
class CacheNeed:
    """What a mixer keeps per token: one or more planes, for all earlier tokens (``window`` 0) or
    for the last ``window`` of them.  Mixers with equal needs share a pool of pages."""
    planes: tuple[CachePlane, ...]
    window: int = 0

    def __post_init__(self):
        names = [p.name for p in self.planes]
        if not names or len(set(names)) != len(names):
            raise ValueError("a cache need has at least one plane, each with a name of its own")

    @property
    def kind(self) -> str:
        return "window" if self.window > 0 else "full"


def keys_and_values(num_kv_heads: int, head_dim: int, window: int = 0) -> CacheNeed:
    """The need of an attention mixer: keys ``k`` stored token by token, values ``v`` stored with
    the tokens of a page innermost (what the attention kernels read in one piece each)."""
    per_token = (int(num_kv_heads), int(head_dim))
    return CacheNeed((CachePlane("k", per_token, "first"), CachePlane("v", per_token, "last")), int(window))


@dataclass(frozen=True)
class StateNeed:
    """What a mixer keeps per request, of fixed size: a tensor of ``shape`` and ``dtype``."""
    shape: tuple[int, ...]
    dtype: str = "float32"
