"""Weights from safetensors, by tensor name.

A model folder holds ``model.safetensors`` (or shards listed by ``model.safetensors.index.json``).
Every tensor the model declares is looked up by its name; before anything is copied to the device
the file is checked against the declarations, and one error lists everything wrong at once:
missing tensors, unexpected tensors, wrong shapes, wrong dtypes (an integer or 64-bit tensor where
the model declares a float one, a float tensor where it declares an integer table).  Tensors the
model does not know are the one thing a file may have too much of: if nothing else is wrong they
are named in a warning and left alone.

Storage on the device: matrices in the engine's dtype (bfloat16, or float32 for the 32-bit path);
tensors declared ``float32`` (norm weights, biases) in 32-bit; integer tables as int32.  A tensor a
checkpoint stores in 32-bit and the model declares ``float32`` therefore stays 32-bit.
"""
from __future__ import annotations

import json
import os
import warnings
from typing import Callable

import torch

from tensorline_amd.parts.spec import TensorDecl

# dtypes of the file (safetensors' names) that a declaration's storage kind accepts
_FLOAT_FILE_DTYPES = {"F32", "F16", "BF16"}
_INT_FILE_DTYPES = {"I32", "I64", "I16", "I8", "U8"}
_ACCEPTED = {"compute": _FLOAT_FILE_DTYPES, "float32": _FLOAT_FILE_DTYPES, "int32": _INT_FILE_DTYPES}


class WeightError(RuntimeError):
    """The checkpoint does not fit the model; ``missing``, ``unexpected``, ``wrong_shape`` and
    ``wrong_dtype`` say how."""

    def __init__(self, path: str, missing: list[str], unexpected: list[str], wrong_shape: list[str],
                 other: list[str] | None = None, wrong_dtype: list[str] | None = None):
        self.path, self.missing, self.unexpected, self.wrong_shape = path, missing, unexpected, wrong_shape
        self.other = other or []
        self.wrong_dtype = wrong_dtype or []
        lines = [f"{path}: the checkpoint does not match the model"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong_shape:
            lines.append(f"  wrong shapes ({len(wrong_shape)}): " + "; ".join(wrong_shape))
        if self.wrong_dtype:
            lines.append(f"  wrong dtypes ({len(self.wrong_dtype)}): " + "; ".join(self.wrong_dtype))
        for o in self.other:
            lines.append("  " + o)
        super().__init__("\n".join(lines))


def checkpoint_files(model_dir: str) -> dict[str, str]:
    """Tensor name -> file, for a single-file or sharded checkpoint."""
    from safetensors import safe_open
    index = os.path.join(model_dir, "model.safetensors.index.json")
    single = os.path.join(model_dir, "model.safetensors")
    names: dict[str, str] = {}
    if os.path.isfile(index):
        with open(index, "r", encoding="utf-8") as f:
            weight_map = json.load(f)["weight_map"]
        for name, fname in weight_map.items():
            names[name] = os.path.join(model_dir, fname)
        return names
    if not os.path.isfile(single):
        raise FileNotFoundError(f"{model_dir}: neither model.safetensors nor model.safetensors.index.json is there")
    with safe_open(single, framework="pt") as f:
        for name in f.keys():
            names[name] = single
    return names


def _target_dtype(decl: TensorDecl, compute: torch.dtype) -> torch.dtype:
    if decl.storage == "compute":
        return compute
    if decl.storage == "float32":
        return torch.float32
    if decl.storage == "int32":
        return torch.int32
    raise ValueError(f"unknown storage kind {decl.storage!r}")


def load_checkpoint(model, model_dir: str, device) -> None:
    """Check ``model_dir`` against ``model.tensor_decls()`` and hand the tensors to the model."""
    from safetensors import safe_open
    model_dir = os.fspath(model_dir)
    decls: dict[str, TensorDecl] = model.tensor_decls()
    optional: dict[str, str] = model.optional_tensors()
    files = checkpoint_files(model_dir)

    handles: dict[str, object] = {}

    def handle(path: str):
        if path not in handles:
            handles[path] = safe_open(path, framework="pt")
        return handles[path]

    missing = sorted(n for n in decls if n not in files)
    unexpected = sorted(n for n in files if n not in decls and n not in optional)
    wrong, wrong_dtype, other = [], [], []
    for name, decl in decls.items():
        if name in files:
            piece = handle(files[name]).get_slice(name)
            shape = tuple(piece.get_shape())
            if shape != tuple(decl.shape):
                wrong.append(f"{name}: file has {list(shape)}, model needs {list(decl.shape)}")
            accepted = _ACCEPTED.get(decl.storage)
            if accepted is None:
                raise ValueError(f"{name}: unknown storage kind {decl.storage!r}")
            file_dtype = str(piece.get_dtype())
            if file_dtype not in accepted:
                wrong_dtype.append(f"{name}: file has {file_dtype}, model needs one of {', '.join(sorted(accepted))}")
    for name, twin in optional.items():
        # e.g. a tied head that the file stores too: it must equal the tensor it is tied to
        if name in files and twin in files:
            a, b = handle(files[name]).get_tensor(name), handle(files[twin]).get_tensor(twin)
            if a.shape != b.shape or not torch.equal(a, b):
                other.append(f"{name} is tied to {twin} but the file holds different values for it")
    if missing or wrong or wrong_dtype or other:
        raise WeightError(model_dir, missing, unexpected, wrong, other, wrong_dtype)
    if unexpected:
        warnings.warn(f"{model_dir}: {len(unexpected)} tensors of the checkpoint are not part of the model and are "
                      "left alone: " + ", ".join(unexpected), stacklevel=2)

    compute = model.dtype

    def get(name: str) -> torch.Tensor:
        t = handle(files[name]).get_tensor(name)
        return t.to(device=device, dtype=_target_dtype(decls[name], compute)).contiguous()

    model.load_tensors(get)


def load_from_getter(model, produce: Callable[[str, TensorDecl], torch.Tensor], device) -> None:
    """Fill a model from a function of (name, declaration), e.g. the random initialiser."""
    decls = model.tensor_decls()
    compute = model.dtype

    def get(name: str) -> torch.Tensor:
        t = produce(name, decls[name])
        if tuple(t.shape) != tuple(decls[name].shape):
            raise WeightError("<generated>", [], [], [f"{name}: got {list(t.shape)}, model needs {list(decls[name].shape)}"])
        return t.to(device=device, dtype=_target_dtype(decls[name], compute)).contiguous()

    model.load_tensors(get)
