"""Engine options, with the names and defaults of the reference's ``BatchEngine`` constructor
(``tensorline/batch_engine.py:79-85``) and of its command line (``tensorline/server.py:256-283``)."""
from __future__ import annotations

from dataclasses import dataclass


@dataclass
class EngineConfig:
    dtype: str = "bfloat16"             # "bfloat16" | "float32" (reference: --dtype, engine.py:59-62)
    block_size: int = 16                 # tokens per KV page (paged.py:110)
    num_blocks: int | None = None        # pages per cache group; None: sized from memory
    kv_mem_fraction: float = 0.6         # share of free HBM for the cache when nothing else is given
    kv_cache_gb: float | None = None     # explicit cache size (batch_engine.py:91-92)
    max_num_seqs: int = 64
    max_batched_tokens: int = 2048       # token budget of one step
    max_model_len: int = 4096
    graphs: bool = True                  # replay pure-decode steps from a HIP graph (--no-cuda-graphs there)
    graph_warmup_tokens: int = 512       # capture graphs for contexts up to this many tokens at start-up
    prefix_caching: bool = True
    overlap: bool = True                 # queue decode step t + 1 before reading step t's tokens (--no-overlap there)
    tune_library: bool = False           # at start-up, let the library pick its kernels by measurement: full prompt portions, decode steps above 64 rows
    device: str = "cuda:0"

    def __post_init__(self):
        self.dtype = normalize_dtype(self.dtype)
        if self.block_size <= 0:
            raise ValueError(f"block_size must be positive, got {self.block_size}")
        if self.max_num_seqs <= 0 or self.max_batched_tokens <= 0 or self.max_model_len <= 1:
            raise ValueError("max_num_seqs, max_batched_tokens must be positive and max_model_len > 1")


def normalize_dtype(name: str) -> str:
    alias = {"bf16": "bfloat16", "bfloat16": "bfloat16", "fp32": "float32", "float32": "float32",
             "float": "float32", "auto": "bfloat16"}
    key = str(name).replace("torch.", "").lower()
    if key not in alias:
        raise ValueError(f"dtype {name!r} is not supported: choose bfloat16 or float32")
    return alias[key]
