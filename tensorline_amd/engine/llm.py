"""The Python entry point: a model folder in, generated tokens out.

The reference's entry points are ``Engine(model_id, device, dtype)`` / ``BatchEngine(model_id,
device, dtype, *, block_size, num_blocks, ...)`` with ``stream(prompt, params, stats)`` and
``abort`` (tensorline/engine.py:55,86-116; tensorline/batch_engine.py:79-85,184-201).  ``LLM`` keeps
those option names and adds ``generate`` for whole batches.  Prompts are lists of token ids, or
text when the model folder has a ``tokenizer.json``.
"""
from __future__ import annotations

import os
import warnings
from dataclasses import dataclass, field
from typing import Iterator, Sequence

import torch

from tensorline_amd.cache.manager import CacheManager
from tensorline_amd.config.engine_config import EngineConfig
from tensorline_amd.engine.detok import IncrementalDetokenizer
from tensorline_amd.engine.engine import InferenceEngine
from tensorline_amd.engine.loading import load_model, random_model
from tensorline_amd.ops import kernels
from tensorline_amd.sampling.params import GenStats, SamplingParams


@dataclass
class RequestOutput:
    token_ids: list[int]
    text: str | None
    finish_reason: str
    stats: GenStats = field(default_factory=GenStats)


class LLM:
    def __init__(self, model: str | os.PathLike | None = None, device: str = "cuda:0", dtype: str = "bfloat16", *,
                 config=None, seed: int = 0, **options):
        """``model``: a folder with config.json and model.safetensors.  Or ``config=`` (a typed
        configuration) with ``seed`` for random weights generated on the GPU.  ``options`` are the
        fields of :class:`EngineConfig` (block_size, num_blocks, kv_cache_gb, max_num_seqs,
        max_batched_tokens, max_model_len, graphs, prefix_caching, ...)."""
        self.config = EngineConfig(dtype=dtype, device=device, **options)
        kernels.require_gpu(device)
        if model is not None:
            self.model, self.model_config = load_model(model, self.config.dtype, device)
            self.tokenizer = _load_tokenizer(model)
        elif config is not None:
            self.model, self.model_config = random_model(config, seed, self.config.dtype, device, generate_on="cuda"), config
            self.tokenizer = None
        else:
            raise ValueError("LLM needs a model folder or a configuration")
        ec = self.config
        max_pos = getattr(self.model_config, "max_position_embeddings", None)
        if max_pos:
            ec.max_model_len = min(ec.max_model_len, int(max_pos))
        num_blocks = ec.num_blocks or self._size_cache()
        if num_blocks * ec.block_size < ec.max_num_seqs * 256:
            warnings.warn(f"KV cache holds only {num_blocks * ec.block_size} tokens ({num_blocks} blocks): "
                          f"{ec.max_num_seqs} concurrent sequences will queue or preempt.", stacklevel=2)
        self.cache = CacheManager(self.model.cache_needs(), self.model.schedule, self.model.state_needs(),
                                  page_size=ec.block_size, num_blocks=num_blocks, max_requests=ec.max_num_seqs,
                                  dtype=self.model.dtype, device=device, prefix_caching=ec.prefix_caching)
        if ec.tune_library and self.model.dtype == torch.bfloat16:
            self.model.tune_library(ec.max_batched_tokens)
        runner = None
        if ec.graphs:
            from tensorline_amd.engine.graphs import GraphRunner
            runner = GraphRunner(self.model, self.cache, max_batch=ec.max_num_seqs,
                                 max_blocks_per_seq=-(-ec.max_model_len // ec.block_size))
            if ec.tune_library and self.model.dtype == torch.bfloat16:
                # decode steps of more rows than the engine's own kernels take are library products too,
                # of exactly the graphs' row counts
                for rows in runner.batch_buckets:
                    if rows > kernels.ROWS64_MAX_ROWS and rows != ec.max_batched_tokens:
                        self.model.tune_library(rows)
            if ec.graph_warmup_tokens:
                runner.warmup(min(ec.graph_warmup_tokens, ec.max_model_len))
        self.engine = InferenceEngine(self.model, self.cache, max_num_seqs=ec.max_num_seqs,
                                      max_batched_tokens=ec.max_batched_tokens, max_model_len=ec.max_model_len,
                                      default_stops=set(self.model.spec.eos_token_ids), runner=runner, overlap=ec.overlap)
        # with or without graphs, every step makes the choices that depend on the longest context alike
        self.engine.runner.fit_context = -(-ec.max_model_len // ec.block_size) * ec.block_size

    def _size_cache(self) -> int:
        """Pages from ``kv_cache_gb`` or from a share of free memory (batch_engine.py:89-97)."""
        ec = self.config
        per_page = CacheManager.bytes_per_page(self.model.cache_needs(), self.model.schedule, ec.block_size,
                                               torch.empty(0, dtype=self.model.dtype).element_size())
        if ec.kv_cache_gb is not None:
            budget = int(ec.kv_cache_gb * (1 << 30))
        else:
            free, _ = torch.cuda.mem_get_info(torch.device(ec.device))
            budget = int(free * ec.kv_mem_fraction)
        # no point in more pages than every sequence at full length can use
        most = ec.max_num_seqs * -(-ec.max_model_len // ec.block_size)
        return max(1, min(budget // max(per_page, 1), most))

    # ---- prompts -------------------------------------------------------------------------------
    def _tokens(self, prompt) -> list[int]:
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise ValueError("text prompts need a tokenizer.json in the model folder; pass token ids instead")
            return self.tokenizer.encode(prompt).ids
        return [int(t) for t in prompt]

    def _text(self, ids: list[int]) -> str | None:
        return self.tokenizer.decode(ids, skip_special_tokens=True) if self.tokenizer is not None else None

    # ---- generation ----------------------------------------------------------------------------
    def generate(self, prompts: Sequence, params: SamplingParams | Sequence[SamplingParams] | None = None) -> list[RequestOutput]:
        """Generate for every prompt, all batched together; outputs in the order of the prompts."""
        if isinstance(prompts, str) or (prompts and isinstance(prompts[0], int)):
            prompts = [prompts]
        plist = list(params) if isinstance(params, (list, tuple)) else [params or SamplingParams()] * len(prompts)
        reqs = [self.engine.add_request(self._tokens(p), sp) for p, sp in zip(prompts, plist)]
        while any(not r.done for r in reqs):
            self.engine.step()
        outs = []
        for r in reqs:
            if r.error is not None:
                raise r.error
            outs.append(RequestOutput(r.output_tokens, self._text(r.output_tokens), r.stats.finish_reason, r.stats))
        return outs

    def stream(self, prompt, params: SamplingParams | None = None, stats: GenStats | None = None) -> Iterator:
        """Yield the request's output as it is produced: text deltas with a tokenizer, token ids
        without.  Other requests that are in flight advance too.  Leaving the generator early aborts
        the request and gives its pages back (batch_engine.py:190-201)."""
        req = self.engine.add_request(self._tokens(prompt), params, stats)
        detok = IncrementalDetokenizer(self.tokenizer) if self.tokenizer is not None else None
        try:
            while not req.done:
                for r, tok in self.engine.step():
                    if r is not req or tok is None:
                        continue
                    if detok is None:
                        yield tok
                    else:
                        delta = detok.push([tok])
                        if delta:
                            yield delta
            if req.error is not None:
                raise req.error
            tail = detok.flush() if detok is not None else ""
            if tail:                                         # the output ended inside a character
                yield tail
        finally:
            self.engine.abort(req)

    def abort(self, req) -> None:
        self.engine.abort(req)

    def counters(self) -> dict:
        return self.engine.counters()


def _load_tokenizer(model_dir):
    path = os.path.join(os.fspath(model_dir), "tokenizer.json")
    if not os.path.isfile(path):
        return None
    from tokenizers import Tokenizer
    return Tokenizer.from_file(path)
