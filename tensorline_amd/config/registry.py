"""One registry from the architecture's name to what builds it.

An :class:`Architecture` ties together the typed configuration class and the function that
turns a configuration into a :class:`tensorline_amd.parts.spec.ModelSpec` (the list of layers
and the order they run in).  The reference gets the same dispatch from
``AutoModelForCausalLM.from_pretrained`` (``tensorline/engine.py:66``).
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Callable

from tensorline_amd.config.model_config import ConfigError


@dataclass(frozen=True)
class Architecture:
    name: str
    config_cls: Any                      # has from_dict(dict) and to_dict()
    build_spec: Callable[[Any], Any]     # config -> ModelSpec


_ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(arch: Architecture, *, replace: bool = False) -> Architecture:
    if arch.name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture {arch.name!r} is already registered")
    _ARCHITECTURES[arch.name] = arch
    return arch


def known_architectures() -> list[str]:
    _ensure_builtin()
    return sorted(_ARCHITECTURES)


def get_architecture(name: str) -> Architecture:
    _ensure_builtin()
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise ConfigError(f"unknown architecture {name!r}; known: {', '.join(sorted(_ARCHITECTURES))}") from None


def architecture_name(cfg_dict: dict) -> str:
    archs = cfg_dict.get("architectures")
    if not archs or not isinstance(archs, (list, tuple)):
        raise ConfigError("config.json: 'architectures' is missing or empty; it selects the model class")
    return str(archs[0])


def load_model_config(model_dir: str | os.PathLike):
    """Read ``<model_dir>/config.json``; return ``(architecture, typed config)``."""
    path = os.path.join(os.fspath(model_dir), "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{path}: no such file (a model folder holds config.json and model.safetensors)")
    with open(path, "r", encoding="utf-8") as f:
        raw = json.load(f)
    arch = get_architecture(architecture_name(raw))
    return arch, arch.config_cls.from_dict(raw)


def _ensure_builtin() -> None:
    # Importing the module registers it; done lazily so that config/ has no import cycle.
    import tensorline_amd.models.qwen2  # noqa: F401
