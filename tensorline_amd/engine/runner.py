"""The step function: runs exactly the tokens it is given, as one batch, from the cache.

``ModelRunner.step(entries)`` takes any mix of prompt portions and single decoded tokens
(:class:`tensorline_amd.engine.batch.StepEntry`), writes their keys and values into the pages the
cache manager holds for each request, and returns float32 logits at the wanted places, in the
order of the entries and of their ``want`` lists (reference: ``PagedModel.forward``,
tensorline/paged.py:190-287).  Generation, trace replay and the benchmark all call this one
function.
"""
from __future__ import annotations

from typing import Sequence

import numpy as np
import torch

from tensorline_amd.cache.manager import CacheManager
from tensorline_amd.engine.batch import LayerCache, PackedBatch, StepContext, StepEntry, pack_batch
from tensorline_amd.models.decoder import DecoderModel


class ModelRunner:
    def __init__(self, model: DecoderModel, cache: CacheManager):
        self.model = model
        self.cache = cache
        self.device = model.device
        self._host: torch.Tensor | None = None       # pinned staging for the step's metadata
        self._dev: torch.Tensor | None = None
        self._copied: torch.cuda.Event | None = None   # recorded after the last copy out of the staging buffer
        self.steps = 0
        self.fit_context = 0          # the longest context this runner's engine allows, if it says so

    # ---- metadata ------------------------------------------------------------------------
    def _upload(self, data: np.ndarray) -> torch.Tensor:
        n = int(data.size)
        pin = torch.device(self.device).type == "cuda"
        if self._dev is None or self._dev.numel() < n:
            if self._copied is not None:
                self._copied.synchronize()
            cap = max(4096, 1 << (max(n, 1) - 1).bit_length())
            self._host = torch.empty(cap, dtype=torch.int32, pin_memory=pin)
            self._dev = torch.empty(cap, dtype=torch.int32, device=self.device)
        if self._copied is not None:
            self._copied.synchronize()    # the last copy out of the staging buffer was only queued: wait before writing it again
        self._host[:n].numpy()[:] = data
        if pin:
            self._dev[:n].copy_(self._host[:n], non_blocking=True)
            if self._copied is None:
                self._copied = torch.cuda.Event()
            self._copied.record()
        else:
            self._dev[:n].copy_(self._host[:n])
        return self._dev

    def _vectors(self, facts) -> dict:
        """Index vectors the model's parts want uploaded with this step; they see the engine's longest context."""
        facts.fit_context = self.fit_context
        fn = getattr(self.model, "step_vectors", None)
        return fn(facts) if fn is not None else {}

    def pack(self, entries: Sequence[StepEntry], pad_seqs: int = 0, pad_nb: Sequence[int] | None = None) -> PackedBatch:
        cache = self.cache
        ngroups = len(cache.groups)
        tables = [[cache.table_array(e.rid, g) for g in range(ngroups)] for e in entries]
        slots = [cache.state_slot(e.rid) for e in entries]
        packed = pack_batch(entries, tables, slots, cache.page_size, ngroups, cache.scratch_page,
                            self.model.vocab_size, pad_seqs=pad_seqs, pad_nb=pad_nb, scratch_slot=cache.scratch_slot,
                            windowed=[g.window > 0 for g in cache.groups], vectors=self._vectors)
        packed.facts.fit_context = self.fit_context
        return packed

    def context(self, packed: PackedBatch, dev: torch.Tensor) -> tuple[StepContext, list[LayerCache]]:
        def view(name: str) -> torch.Tensor:
            off, n = packed.offsets[name]
            return dev[off:off + n]

        ctx = StepContext(
            num_tokens=packed.T, num_seqs=packed.S, ids=view("ids"), pos=view("pos"),
            seq_of_token=view("seq_of_token"), q_start=view("q_start"), ctx_start=view("ctx_start"),
            state_slots=view("state_slots"), logit_rows=view("logit_rows"), facts=packed.facts,
            host_q_start=packed.host_q_start, host_ctx_start=packed.host_ctx_start,
            host_state_slots=packed.host_state_slots, logits_for_all_rows=packed.logits_for_all_rows,
            extra={name[6:]: view(name) for name in packed.offsets if name.startswith("extra:")})
        cache = self.cache
        g_slots = [view(f"slots{g}") for g in range(len(cache.groups))]
        g_tables = [view(f"tables{g}").view(packed.S, packed.group_nb[g]) for g in range(len(cache.groups))]
        views: list[LayerCache] = []
        for i in range(len(self.model.schedule)):
            g = cache.group_of_entry[i]
            views.append(LayerCache(
                planes=cache.storage(i), slots=g_slots[g] if g is not None else None,
                tables=g_tables[g] if g is not None else None,
                write=cache.owns_storage(i), state=cache.state.get(i)))
        return ctx, views

    # ---- one step ------------------------------------------------------------------------
    @staticmethod
    def _take_tokens(dev: torch.Tensor, packed: PackedBatch, token_source: torch.Tensor) -> None:
        """Overwrite the step's token ids on the device with ``token_source`` (int32, a token per
        entry in the order of the entries): the step then runs on tokens the host has not seen yet."""
        if packed.T != packed.S:
            raise ValueError("tokens can be taken from the device only for steps of one token per request")
        off, _ = packed.offsets["ids"]
        n = token_source.numel()
        dev[off:off + n].copy_(token_source, non_blocking=True)

    @torch.inference_mode()
    def step(self, entries: Sequence[StepEntry], token_source: torch.Tensor | None = None) -> torch.Tensor:
        """Logits [number of wanted places, vocab] in float32.  ``token_source``: see ``_take_tokens``."""
        packed = self.pack(entries)
        dev = self._upload(packed.data)
        if token_source is not None:
            self._take_tokens(dev, packed, token_source)
        ctx, views = self.context(packed, dev)
        self.steps += 1
        return self.model.forward(ctx, views)
