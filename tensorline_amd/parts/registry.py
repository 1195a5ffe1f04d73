"""Registries of part kinds.  A kind maps to a class; a model names kinds in its spec.

New parts register themselves with the decorators below; nothing else in the framework has to
change to use them in a :class:`tensorline_amd.parts.spec.ModelSpec`.
"""
from __future__ import annotations

from typing import Callable

from tensorline_amd.parts.spec import PartSpec

MIXERS: dict[str, type] = {}
FEED_FORWARDS: dict[str, type] = {}
NORMS: dict[str, type] = {}
POSITIONS: dict[str, type] = {}
BLOCKS: dict[str, type] = {}
EMBEDDINGS: dict[str, type] = {}
HEADS: dict[str, type] = {}

_TABLES = {"mixer": MIXERS, "feed_forward": FEED_FORWARDS, "norm": NORMS, "position": POSITIONS, "block": BLOCKS,
           "embedding": EMBEDDINGS, "head": HEADS}


def _register(table: dict[str, type], what: str, kind: str, replace: bool) -> Callable[[type], type]:
    def deco(cls: type) -> type:
        if kind in table and not replace:
            raise ValueError(f"{what} kind {kind!r} is already registered")
        table[kind] = cls
        return cls
    return deco


def register_mixer(kind: str, replace: bool = False):
    return _register(MIXERS, "mixer", kind, replace)


def register_feed_forward(kind: str, replace: bool = False):
    return _register(FEED_FORWARDS, "feed-forward", kind, replace)


def register_norm(kind: str, replace: bool = False):
    return _register(NORMS, "norm", kind, replace)


def register_position(kind: str, replace: bool = False):
    return _register(POSITIONS, "position encoding", kind, replace)


def register_block(kind: str, replace: bool = False):
    return _register(BLOCKS, "block", kind, replace)


def register_embedding(kind: str, replace: bool = False):
    return _register(EMBEDDINGS, "embedding", kind, replace)


def register_head(kind: str, replace: bool = False):
    return _register(HEADS, "head", kind, replace)


def build_part(what: str, spec: PartSpec, layer_prefix: str | None = None, **common):
    """Instantiate the part ``spec`` names: ``cls(**common, **spec.params)``; parts that read
    checkpoint tensors get ``prefix = layer_prefix + spec.prefix``."""
    _ensure_builtin()
    if layer_prefix is not None:
        common["prefix"] = layer_prefix + spec.prefix
    table = _TABLES[what]
    try:
        cls = table[spec.kind]
    except KeyError:
        raise ValueError(f"unknown {what} kind {spec.kind!r}; known: {', '.join(sorted(table))}") from None
    return cls(**common, **spec.params)


def _ensure_builtin() -> None:
    import tensorline_amd.parts.attention  # noqa: F401
    import tensorline_amd.parts.block  # noqa: F401
    import tensorline_amd.parts.embedding  # noqa: F401
    import tensorline_amd.parts.feedforward  # noqa: F401
    import tensorline_amd.parts.norm  # noqa: F401
    import tensorline_amd.parts.rotary  # noqa: F401
