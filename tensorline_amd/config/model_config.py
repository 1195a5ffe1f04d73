"""Typed model configuration for the dense Qwen2.5 decoder.

Every size and constant of the model comes from ``config.json`` through this
dataclass; no other module hard-codes one.  The reference engine reads the same
keys through the Hugging Face config object (``tensorline/paged.py:113-119``,
``tensorline/manager.py:46-54``): ``num_attention_heads``,
``num_key_value_heads``, ``head_dim`` (falling back to ``hidden_size //
num_attention_heads``), ``hidden_size``, ``intermediate_size``,
``num_hidden_layers``, ``vocab_size`` and ``tie_word_embeddings``.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field, fields
from typing import Any, Mapping


class ConfigError(ValueError):
    """A ``config.json`` that this engine cannot serve, with the reason."""


def _require(d: Mapping[str, Any], key: str, kind=int):
    if key not in d or d[key] is None:
        raise ConfigError(f"config.json: required key '{key}' is missing")
    v = d[key]
    if kind is int:
        if isinstance(v, bool) or not isinstance(v, int):
            raise ConfigError(f"config.json: '{key}' must be an integer, got {v!r}")
        if v <= 0:
            raise ConfigError(f"config.json: '{key}' must be positive, got {v}")
    return v


@dataclass(frozen=True)
class Qwen2Config:
    """``Qwen2ForCausalLM``: GQA attention with q/k/v bias, rotate-half RoPE,
    RMSNorm, SwiGLU feed-forward, tied or untied output head."""

    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float = 1e-6
    rope_theta: float = 10000.0
    tie_word_embeddings: bool = False
    max_position_embeddings: int = 32768
    hidden_act: str = "silu"
    attention_bias: bool = True          # q/k/v carry a bias, o does not (tests/test_batching.py:48)
    eos_token_id: tuple[int, ...] = ()
    bos_token_id: int | None = None
    architecture: str = "Qwen2ForCausalLM"
    extra: Mapping[str, Any] = field(default_factory=dict, compare=False, hash=False)

    # ---- derived -----------------------------------------------------------------------
    @property
    def group_size(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    @property
    def q_size(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_key_value_heads * self.head_dim

    # ---- construction ------------------------------------------------------------------
    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "Qwen2Config":
        archs = d.get("architectures") or []
        arch = archs[0] if archs else d.get("architecture", "Qwen2ForCausalLM")
        hidden = _require(d, "hidden_size")
        nq = _require(d, "num_attention_heads")
        nkv = d.get("num_key_value_heads")
        nkv = nq if nkv is None else _require(d, "num_key_value_heads")
        head_dim = d.get("head_dim")
        if head_dim is None:
            if hidden % nq:
                raise ConfigError(
                    f"config.json: hidden_size {hidden} is not a multiple of num_attention_heads {nq} "
                    "and no head_dim is given")
            head_dim = hidden // nq
        else:
            head_dim = _require(d, "head_dim")
        eos = d.get("eos_token_id")
        if eos is None:
            eos_ids: tuple[int, ...] = ()
        elif isinstance(eos, (list, tuple)):
            eos_ids = tuple(int(e) for e in eos)
        else:
            eos_ids = (int(eos),)
        known = {f.name for f in fields(cls)} | {
            "architectures", "torch_dtype", "dtype", "model_type", "transformers_version", "use_cache",
            "use_sliding_window", "sliding_window", "max_window_layers", "rope_scaling",
            "initializer_range", "attention_dropout", "layer_types"}
        cfg = cls(
            vocab_size=_require(d, "vocab_size"),
            hidden_size=hidden,
            intermediate_size=_require(d, "intermediate_size"),
            num_hidden_layers=_require(d, "num_hidden_layers"),
            num_attention_heads=nq,
            num_key_value_heads=nkv,
            head_dim=head_dim,
            rms_norm_eps=float(d.get("rms_norm_eps", 1e-6)),
            rope_theta=float(d.get("rope_theta", 10000.0)),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            max_position_embeddings=int(d.get("max_position_embeddings", 32768)),
            hidden_act=str(d.get("hidden_act", "silu")),
            attention_bias=bool(d.get("attention_bias", True)),
            eos_token_id=eos_ids,
            bos_token_id=d.get("bos_token_id"),
            architecture=arch,
            extra={k: v for k, v in d.items() if k not in known},
        )
        cfg._check_unsupported(d)
        cfg.validate()
        return cfg

    @classmethod
    def from_json(cls, path: str | os.PathLike) -> "Qwen2Config":
        p = os.fspath(path)
        if os.path.isdir(p):
            p = os.path.join(p, "config.json")
        with open(p, "r", encoding="utf-8") as f:
            return cls.from_dict(json.load(f))

    # ---- validation --------------------------------------------------------------------
    @staticmethod
    def _check_unsupported(d: Mapping[str, Any]) -> None:
        # The reference never reads these keys: a checkpoint that needs them would be
        # served wrongly, so it is refused instead.
        if d.get("use_sliding_window"):
            raise ConfigError("config.json: use_sliding_window=true is not supported for Qwen2ForCausalLM "
                              "(the reference attends to all keys, tensorline/paged.py:237)")
        if d.get("rope_scaling") not in (None, {}):
            raise ConfigError(f"config.json: rope_scaling={d['rope_scaling']!r} is not supported")

    def validate(self) -> None:
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"config.json: num_attention_heads {self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"config.json: head_dim {self.head_dim} must be even for rotate-half RoPE")
        if self.hidden_act != "silu":
            raise ConfigError(f"config.json: hidden_act {self.hidden_act!r} is not supported (only 'silu')")
        if not (self.rms_norm_eps >= 0.0):
            raise ConfigError(f"config.json: rms_norm_eps {self.rms_norm_eps} must be >= 0")
        if not (self.rope_theta > 0.0):
            raise ConfigError(f"config.json: rope_theta {self.rope_theta} must be > 0")
        if self.max_position_embeddings <= 0:
            raise ConfigError("config.json: max_position_embeddings must be positive")

    # ---- output ------------------------------------------------------------------------
    def to_dict(self) -> dict[str, Any]:
        """The ``config.json`` contents that reproduce this configuration."""
        out: dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": "qwen2",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "tie_word_embeddings": self.tie_word_embeddings,
            "max_position_embeddings": self.max_position_embeddings,
            "hidden_act": self.hidden_act,
            "attention_bias": self.attention_bias,
            "use_sliding_window": False,
        }
        if self.eos_token_id:
            out["eos_token_id"] = list(self.eos_token_id) if len(self.eos_token_id) > 1 else self.eos_token_id[0]
        if self.bos_token_id is not None:
            out["bos_token_id"] = self.bos_token_id
        return out
