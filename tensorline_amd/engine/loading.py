"""From a model folder (or a configuration and a seed) to a model with its weights on the GPU."""
from __future__ import annotations

import os

import torch

from tensorline_amd.config.engine_config import normalize_dtype
from tensorline_amd.config.registry import get_architecture, load_model_config
from tensorline_amd.models.decoder import DecoderModel
from tensorline_amd.weights.loader import load_checkpoint, load_from_getter
from tensorline_amd.weights.random_init import random_tensor

TORCH_DTYPE = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def load_model(model_dir: str | os.PathLike, dtype: str = "bfloat16", device="cuda:0"):
    """Read config.json, pick the architecture by name, build the model and load its weights.
    Returns ``(model, config)``."""
    arch, config = load_model_config(model_dir)
    model = DecoderModel(arch.build_spec(config), TORCH_DTYPE[normalize_dtype(dtype)], device)
    load_checkpoint(model, os.fspath(model_dir), device)
    return model, config


def random_model(config, seed: int = 0, dtype: str = "bfloat16", device="cuda:0", generate_on: str | None = None):
    """A model of ``config`` with random weights.  ``generate_on="cpu"`` draws the same values as
    :func:`tensorline_amd.weights.random_init.write_random_model`; drawing on the GPU is faster for
    large models and gives other (equally distributed) values."""
    arch = get_architecture(config.architecture)
    model = DecoderModel(arch.build_spec(config), TORCH_DTYPE[normalize_dtype(dtype)], device)
    gen_dev = generate_on or "cpu"
    load_from_getter(model, lambda name, decl: random_tensor(name, decl, seed, gen_dev), device)
    return model
