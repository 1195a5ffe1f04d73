"""One step's batch: what the caller hands in and the flat device metadata built from it.

A step takes, per request, its next tokens: a whole prompt, a portion of one cut anywhere, or a
single decoded token, in any mix (reference: ``SeqChunk`` and the flattening in
tensorline/paged.py:100-106,194-238).  All index data of a step is packed into one int32 vector
and copied to the device once; the kernels read views of it.  Nothing here knows what a mixer
caches or how it launches its kernels: a part that wants an index list of its own on the device
computes it from the step's facts (``step_vectors``) and finds it in ``StepContext.extra``.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Sequence

import numpy as np
import torch


@dataclass
class StepEntry:
    """``tokens`` are the request's next tokens, at positions ``start .. start+len-1``; ``start``
    tokens are already in the cache.  ``want`` lists the places among ``tokens`` whose logits are
    asked for (the reference asks for the last one only: ``want_logits``)."""
    rid: object
    tokens: Sequence[int]
    start: int
    want: Sequence[int] = ()


@dataclass
class StepFacts:
    """What the host knows about the step's shape.  Parts choose their launches from it; nothing in
    it belongs to one kind of part."""
    max_context: int = 0          # largest start + len over the step's sequences
    max_query_len: int = 0        # largest number of tokens one sequence brings
    decode_only: bool = False     # every sequence brings exactly one token
    num_seqs: int = 0             # sequences of the step, padding sequences (one token each, after the real ones) included
    q_lens: list[int] = field(default_factory=list)    # tokens each real sequence brings
    starts: list[int] = field(default_factory=list)    # tokens each real sequence has cached already
    # The longest context the engine will ever run, if the caller knows it (0: unknown).  Choices
    # that must be the same in every step of an engine are made for it.
    fit_context: int = 0


@dataclass
class LayerCache:
    """The cache as one schedule entry sees it in this step."""
    planes: dict[str, torch.Tensor]   # the pages of each plane its mixer declared, by name
    slots: torch.Tensor | None        # int32 [T]: cache row of each token of the step
    tables: torch.Tensor | None       # int32 [S, NB]: page ids of each sequence
    write: bool                       # False: the entry reads a cache another entry wrote
    state: torch.Tensor | None = None  # [slots + 1, *shape] fixed-size per-request state, if any


@dataclass
class StepContext:
    num_tokens: int
    num_seqs: int
    ids: torch.Tensor                 # int32 [T]
    pos: torch.Tensor                 # int32 [T]
    seq_of_token: torch.Tensor        # int32 [T]
    q_start: torch.Tensor             # int32 [S + 1]: first row of each sequence in the flat batch
    ctx_start: torch.Tensor           # int32 [S]: tokens of the sequence already cached
    state_slots: torch.Tensor         # int32 [S]
    logit_rows: torch.Tensor          # int32 [R]
    facts: StepFacts
    # int32 vectors that parts asked to have uploaded with the step (``step_vectors``), by name
    extra: dict[str, torch.Tensor] = field(default_factory=dict)
    # host mirrors, for parts that loop over sequences on the host
    host_q_start: list[int] = field(default_factory=list)
    host_ctx_start: list[int] = field(default_factory=list)
    host_state_slots: list[int] = field(default_factory=list)
    logits_for_all_rows: bool = False  # logit_rows is 0, 1, .., T-1: no gather is needed


@dataclass
class PackedBatch:
    """The int32 vector of one step and where its pieces lie."""
    data: np.ndarray
    T: int
    S: int
    R: int
    offsets: dict[str, tuple[int, int]]
    group_nb: list[int]
    facts: StepFacts
    host_q_start: list[int]
    host_ctx_start: list[int]
    host_state_slots: list[int]
    logits_for_all_rows: bool = False


def pack_batch(entries: Sequence[StepEntry], tables: Sequence[Sequence[Sequence[int]]], state_slots: Sequence[int],
               page_size: int, num_groups: int, scratch_page: int, vocab_size: int,
               pad_seqs: int = 0, pad_nb: Sequence[int] | None = None, scratch_slot: int = 0,
               windowed: Sequence[bool] | None = None, vectors=None) -> PackedBatch:
    """Flatten a step.  ``tables[s][g]`` is the page table of sequence ``s`` in group ``g`` and must
    cover positions < start + len.  With ``pad_seqs``/``pad_nb`` the batch is padded to a fixed
    shape with one-token rows that touch only the scratch page and the scratch slot.
    ``vectors``: a function from the step's :class:`StepFacts` to int32 vectors by name (index lists
    that parts want on the device for this step); they travel in the same upload."""
    S = len(entries)
    if S == 0:
        raise ValueError("a step needs at least one entry")
    if windowed is None:
        windowed = [True] * num_groups               # assume tables may hold pages already given back
    q_lens = [len(e.tokens) for e in entries]
    if min(q_lens) <= 0:
        raise ValueError("every entry of a step brings at least one token")
    S_pad = max(S, pad_seqs)
    T_real = sum(q_lens)
    T = T_real + (S_pad - S)
    ids = np.empty(T, np.int32)
    pos = np.empty(T, np.int32)
    seq_of = np.empty(T, np.int32)
    q_start = np.empty(S_pad + 1, np.int32)
    ctx_start = np.zeros(S_pad, np.int32)
    slots_state = np.full(S_pad, scratch_slot, np.int32)
    rows: list[int] = []

    group_nb = []
    for g in range(num_groups):
        nb = max(len(tables[s][g]) for s in range(S))
        if pad_nb is not None:
            if nb > pad_nb[g]:
                raise ValueError(f"page table of {nb} entries exceeds the fixed width {pad_nb[g]}")
            nb = pad_nb[g]
        group_nb.append(max(nb, 1))
    g_slots = [np.full(T, scratch_page * page_size, np.int32) for _ in range(num_groups)]
    g_tables = [np.full((S_pad, group_nb[g]), scratch_page, np.int32) for g in range(num_groups)]

    r0 = 0
    for s, e in enumerate(entries):
        n = q_lens[s]
        if e.start < 0:
            raise ValueError(f"request {e.rid!r}: negative start")
        need_pages = -(-(e.start + n) // page_size)
        if n == 1:                                   # a decoded token: scalars instead of arrays
            tok = int(e.tokens[0])
            if not 0 <= tok < vocab_size:
                raise ValueError(f"request {e.rid!r}: token id outside [0, {vocab_size})")
            ids[r0] = tok
            pos[r0] = e.start
            p = None
        else:
            toks = np.asarray(e.tokens, dtype=np.int64)
            if toks.min() < 0 or toks.max() >= vocab_size:
                raise ValueError(f"request {e.rid!r}: token id outside [0, {vocab_size})")
            ids[r0:r0 + n] = toks
            p = np.arange(e.start, e.start + n, dtype=np.int32)
            pos[r0:r0 + n] = p
        seq_of[r0:r0 + n] = s
        q_start[s] = r0
        ctx_start[s] = e.start
        slots_state[s] = state_slots[s]
        for g in range(num_groups):
            tab = tables[s][g]
            if not isinstance(tab, np.ndarray):
                tab = np.asarray(tab, dtype=np.int32)
            if len(tab) < need_pages:
                raise ValueError(f"request {e.rid!r}: page table covers {len(tab) * page_size} tokens, "
                                 f"{e.start + n} are needed")
            if p is None:
                page = int(tab[e.start // page_size])
                if page < 0:
                    raise ValueError(f"request {e.rid!r}: a token of this step lies on a page already given back")
                g_slots[g][r0] = page * page_size + e.start % page_size
            else:
                pages = tab[p // page_size]
                if pages.min() < 0:
                    raise ValueError(f"request {e.rid!r}: a token of this step lies on a page already given back")
                g_slots[g][r0:r0 + n] = pages * page_size + p % page_size
            row = g_tables[g][s]
            row[:len(tab)] = tab
            if windowed[g]:                          # pages a window has passed: any valid page will do
                np.putmask(row[:len(tab)], tab < 0, scratch_page)
        for w in e.want:
            if not 0 <= w < n:
                raise ValueError(f"request {e.rid!r}: wanted place {w} is outside its {n} tokens")
            rows.append(r0 + int(w))
        r0 += n
    # padding rows: token 0 at position 0 of a sequence that lives on the scratch page
    for s in range(S, S_pad):
        ids[r0] = 0
        pos[r0] = 0
        seq_of[r0] = s
        q_start[s] = r0
        rows.append(r0)           # a fixed-shape batch has a logits row for every sequence
        r0 += 1
    q_start[S_pad] = r0

    pieces: list[tuple[str, np.ndarray]] = [
        ("ids", ids), ("pos", pos), ("seq_of_token", seq_of), ("q_start", q_start), ("ctx_start", ctx_start),
        ("state_slots", slots_state), ("logit_rows", np.asarray(rows, np.int32))]
    starts = [e.start for e in entries]
    facts = StepFacts(
        max_context=max(st + n for st, n in zip(starts, q_lens)), max_query_len=max(q_lens),
        decode_only=all(n == 1 for n in q_lens), num_seqs=S_pad, q_lens=q_lens, starts=starts)
    extra = vectors(facts) if vectors is not None else {}
    for name in sorted(extra):
        pieces.append(("extra:" + name, np.asarray(extra[name], np.int32).reshape(-1)))
    for g in range(num_groups):
        pieces.append((f"slots{g}", g_slots[g]))
        pieces.append((f"tables{g}", g_tables[g].reshape(-1)))
    offsets, off = {}, 0
    for name, arr in pieces:
        offsets[name] = (off, arr.size)
        off += arr.size
    data = np.concatenate([a for _, a in pieces]) if off else np.zeros(0, np.int32)
    return PackedBatch(data.astype(np.int32, copy=False), T, S_pad, len(rows), offsets, group_nb, facts,
                       [int(v) for v in q_start], [int(v) for v in ctx_start], [int(v) for v in slots_state],
                       logits_for_all_rows=rows == list(range(T)))
