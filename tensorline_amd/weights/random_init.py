"""Random weights from a configuration and a seed, and the model folder written from them.

Each tensor has a generator of its own, seeded by (seed, tensor name), so a tensor's values do
not depend on which others exist.  Values are drawn in float32 and rounded to bfloat16 before
they are stored, so the 32-bit and the bfloat16 engine read identical numbers.  Scheme: matrices,
embeddings and biases N(0, 0.02); norm weights 1 + N(0, 0.1).
"""
from __future__ import annotations

import hashlib
import json
import os

import torch

from tensorline_amd.parts.spec import TensorDecl


def _tensor_seed(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") & ((1 << 63) - 1)


def random_tensor(name: str, decl: TensorDecl, seed: int, device="cpu", round_to_bf16: bool = True) -> torch.Tensor:
    """The tensor ``name`` of the random model ``seed``, in float32 (int32 for integer tables).
    The values depend on the kind of device the generator runs on."""
    dev = torch.device(device)
    gen = torch.Generator(device=dev)
    gen.manual_seed(_tensor_seed(seed, name))
    if decl.storage == "int32":
        return torch.zeros(decl.shape, dtype=torch.int32, device=dev)
    t = torch.randn(decl.shape, generator=gen, dtype=torch.float32, device=dev)
    if decl.init == "normal":
        t.mul_(decl.std)
    elif decl.init == "one_plus_normal":
        t.mul_(decl.std).add_(1.0)
    elif decl.init == "zeros":
        t.zero_()
    else:
        raise ValueError(f"{name}: unknown init {decl.init!r}")
    if round_to_bf16:
        t = t.to(torch.bfloat16).to(torch.float32)
    return t


def write_random_model(config, out_dir: str, seed: int = 0, store_dtype: str = "bfloat16") -> str:
    """Write ``config.json`` and ``model.safetensors`` for a random model of ``config`` (a typed
    configuration of a registered architecture).  Returns ``out_dir``."""
    from safetensors.torch import save_file

    from tensorline_amd.config.registry import get_architecture
    from tensorline_amd.models.decoder import DecoderModel

    arch = get_architecture(config.architecture)
    spec = arch.build_spec(config)
    model = DecoderModel(spec, torch.float32, "cpu")
    store = {"bfloat16": torch.bfloat16, "float32": torch.float32}[store_dtype]
    tensors = {}
    for name, decl in model.tensor_decls().items():
        t = random_tensor(name, decl, seed, "cpu")
        tensors[name] = t if decl.storage == "int32" else t.to(store).contiguous()
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(config.to_dict(), f, indent=1)
    save_file(tensors, os.path.join(out_dir, "model.safetensors"), metadata={"format": "pt", "seed": str(seed)})
    return out_dir
