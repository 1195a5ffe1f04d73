"""The cache manager: paged keys and values per group of layers, page tables per request, and
slots for fixed-size per-request state.

* **Groups.**  Schedule entries whose mixers keep the same thing per token (the same planes, see
  :class:`tensorline_amd.parts.spec.CacheNeed`, and the same window) form a group.  What a plane
  means (keys, values, something else) is the mixer's business: the manager allocates
  ``[pages, page, *shape]`` or ``[pages, *shape, page]`` per plane and entry, and hands them out by name.  A group has its own page pool: its own page ids and one
  allocator; within a group one page id addresses the same page in every member's storage
  (reference: one id for all layers, tensorline/paged.py:128-130).  An entry that reads another
  entry's cache belongs to that entry's group and has no storage of its own.
* **Tables.**  Per request and group, a list indexed by logical page (position // page size)
  holding the physical page id, or -1 once a windowed group has given the page back.
* **Giving back.**  ``release`` returns everything when a request ends, is aborted or
  preempted (tensorline/batch_engine.py:261-264); ``trim`` returns the pages of a windowed group
  that no later token can see.  Returned pages are handed out again; nothing is zeroed: lengths
  and tables keep stale contents invisible.
* **State slots.**  Each live request owns one slot index into per-entry state arenas
  ``[max_requests + 1, *shape]`` (the last slot is scratch for padding rows).  A slot's state is
  zeroed when it is handed out.  This architecture has no such state; the slots exist anyway.
* **Scratch page.**  Page ``num_blocks`` of every storage is outside the allocator: padding rows
  of fixed-shape decode batches write there (tensorline/paged.py:125-128).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Sequence

import numpy as np
import torch

from tensorline_amd.cache.allocator import PagePool, page_key
from tensorline_amd.parts.spec import CacheNeed, ScheduleEntry, StateNeed

_TORCH_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32}


def _plane_dtype(name: str, compute: torch.dtype) -> torch.dtype:
    return compute if name == "compute" else _TORCH_DTYPES[name]


@dataclass
class CacheGroup:
    need: CacheNeed
    entries: list[int]                       # schedule entries with storage in this group
    allocator: PagePool
    storage: dict[int, dict[str, torch.Tensor]] = field(default_factory=dict)   # entry -> plane name -> pages

    @property
    def window(self) -> int:
        return self.need.window


@dataclass
class _Request:
    tables: list[list[int]]                  # per group: logical page -> physical page or -1
    trimmed: list[int]                       # per group: logical pages below this are given back
    state_slot: int
    hashes: list[int] = field(default_factory=list)   # content hashes of its full, computed pages
    arrays: list = field(default_factory=list)        # per group: the table as an int32 array, or None when stale
    serial: int = 0                                   # which admission of the request this is (never reused)


class CacheManager:
    def __init__(self, cache_needs: Sequence[CacheNeed | None], schedule: Sequence[ScheduleEntry],
                 state_needs: Sequence[StateNeed | None], *, page_size: int, num_blocks: int, max_requests: int,
                 dtype: torch.dtype, device, prefix_caching: bool = False, allocate_storage: bool = True):
        if page_size <= 0 or num_blocks <= 0 or max_requests <= 0:
            raise ValueError("page_size, num_blocks and max_requests must be positive")
        self.page_size, self.num_blocks, self.max_requests = page_size, num_blocks, max_requests
        self.dtype, self.device = dtype, device
        self.scratch_page = num_blocks
        self.scratch_slot = max_requests

        # ---- groups ----
        self.groups: list[CacheGroup] = []
        self.group_of_entry: list[int | None] = [None] * len(schedule)
        self.storage_entry: list[int | None] = [None] * len(schedule)
        by_need: dict[CacheNeed, int] = {}
        for i, (e, need) in enumerate(zip(schedule, cache_needs)):
            if need is None:
                continue
            if e.cache_from is not None:
                src = e.cache_from
                src_need = cache_needs[src]
                if src_need is None or src_need.planes != need.planes:
                    raise ValueError(f"schedule entry {i} reads the cache of entry {src}, which keeps something else per token")
                self.group_of_entry[i] = self.group_of_entry[src]
                self.storage_entry[i] = src
                continue
            g = by_need.get(need)
            if g is None:
                g = len(self.groups)
                by_need[need] = g
                self.groups.append(CacheGroup(need, [], PagePool(num_blocks, share_prefixes=False)))
            self.groups[g].entries.append(i)
            self.group_of_entry[i] = g
            self.storage_entry[i] = i
        self._windowed = any(g.window > 0 for g in self.groups)
        self._serial = 0
        # an entry that reads a windowed entry's cache with a wider view would see freed pages
        for i, e in enumerate(schedule):
            if e.cache_from is not None and cache_needs[i] is not None:
                src_w, my_w = cache_needs[e.cache_from].window, cache_needs[i].window
                if src_w > 0 and (my_w == 0 or my_w > src_w):
                    raise ValueError(f"schedule entry {i} looks further back than the cache of entry {e.cache_from} keeps")

        # ---- state slots ----
        self.state_needs = list(state_needs)
        self.has_state = any(n is not None for n in self.state_needs)
        self._free_slots: list[int] = list(range(max_requests - 1, -1, -1))
        self.state: dict[int, torch.Tensor] = {}

        # prefix sharing: only where one page id means the same tokens for every layer and no
        # mixer carries state that pages do not hold
        self.prefix_caching = bool(prefix_caching) and len(self.groups) == 1 and self.groups[0].window == 0 \
            and not self.has_state
        if self.prefix_caching:
            self.groups[0].allocator.share_prefixes = True

        if allocate_storage:
            for g in self.groups:
                for i in g.entries:                       # one page more than the pool: the scratch page
                    g.storage[i] = {
                        plane.name: torch.zeros(plane.storage_shape(num_blocks + 1, page_size),
                                                dtype=_plane_dtype(plane.dtype, dtype), device=device)
                        for plane in g.need.planes}
            for i, need in enumerate(self.state_needs):
                if need is not None:
                    self.state[i] = torch.zeros((max_requests + 1, *need.shape), dtype=_TORCH_DTYPES[need.dtype], device=device)

        self._requests: dict[object, _Request] = {}

    # ---- sizes ---------------------------------------------------------------------------
    @staticmethod
    def bytes_per_page(cache_needs: Sequence[CacheNeed | None], schedule: Sequence[ScheduleEntry], page_size: int,
                       elem_size: int) -> int:
        """Bytes one page id costs over all entries with storage: every plane of every such entry
        (keys and values of each layer in the reference: tensorline/paged.py:132-137).  ``elem_size``
        is that of the cache's own dtype."""
        total = 0
        for e, need in zip(schedule, cache_needs):
            if need is not None and e.cache_from is None:
                for plane in need.planes:
                    size = elem_size if plane.dtype == "compute" else torch.empty(0, dtype=_TORCH_DTYPES[plane.dtype]).element_size()
                    total += page_size * plane.values_per_token() * size
        return total

    def pages_for(self, tokens: int) -> int:
        return -(-tokens // self.page_size)

    def num_free(self, group: int = 0) -> int:
        return self.groups[group].allocator.num_free

    def min_free(self) -> int:
        return min((g.allocator.num_free for g in self.groups), default=self.num_blocks)

    def all_free(self) -> bool:
        """No page and no slot is held (reference invariant: tests/test_batching.py:80)."""
        return all(g.allocator.num_free == g.allocator.num_pages for g in self.groups) \
            and len(self._free_slots) == self.max_requests and not self._requests

    def can_ever_hold(self, tokens: int, step_tokens: int) -> bool:
        """Could a request of ``tokens`` tokens be held if it were alone?  A windowed group needs
        pages for its window plus one step's portion only."""
        for g in self.groups:
            if g.window > 0:
                span = min(tokens, g.window + step_tokens + self.page_size)
            else:
                span = tokens
            if self.pages_for(span) > self.num_blocks:
                return False
        return True

    # ---- requests ------------------------------------------------------------------------
    def has_request(self, rid) -> bool:
        return rid in self._requests

    def free_slots(self) -> int:
        return len(self._free_slots)

    def add_request(self, rid) -> int | None:
        """Give the request a state slot (zeroed) and empty tables; None if no slot is free."""
        if rid in self._requests:
            raise KeyError(f"request {rid!r} is already live")
        if not self._free_slots:
            return None
        slot = self._free_slots.pop()
        for t in self.state.values():
            t[slot].zero_()
        self._serial += 1
        self._requests[rid] = _Request([[] for _ in self.groups], [0] * len(self.groups), slot,
                                       arrays=[None] * len(self.groups), serial=self._serial)
        return slot

    @property
    def has_windows(self) -> bool:
        """Whether some group gives pages back while a request lives (a windowed group)."""
        return self._windowed

    def admission(self, rid) -> int:
        """A number that differs between two admissions of a request id (its pages were given back
        in between): whoever keeps a copy of a table can tell that it is stale."""
        return self._requests[rid].serial

    def state_slot(self, rid) -> int:
        return self._requests[rid].state_slot

    def table(self, rid, group: int = 0) -> list[int]:
        return self._requests[rid].tables[group]

    def table_array(self, rid, group: int = 0) -> np.ndarray:
        """The table as an int32 array, rebuilt only after it changed (a step of a large batch would
        otherwise convert every list again)."""
        req = self._requests[rid]
        arr = req.arrays[group]
        if arr is None:
            arr = req.arrays[group] = np.asarray(req.tables[group], dtype=np.int32)
        return arr

    def grow(self, rid, upto: int) -> bool:
        """Make every group's table cover positions < ``upto``.  All groups or none
        (reference ``_grow``: tensorline/batch_engine.py:251-259)."""
        req = self._requests[rid]
        want = self.pages_for(upto)
        if all(len(t) >= want for t in req.tables):          # the usual case of a decoded token: nothing to add
            return True
        needs = [max(0, want - len(t)) for t in req.tables]
        if any(n > g.allocator.num_free for n, g in zip(needs, self.groups)):
            return False
        for gi, (n, g, t) in enumerate(zip(needs, self.groups, req.tables)):
            if n:
                got = g.allocator.take(n)
                assert got is not None
                t.extend(got)
                req.arrays[gi] = None
        return True

    def trim(self, rid, computed: int) -> int:
        """After ``computed`` tokens are cached: give back the pages of windowed groups that hold
        only positions no later token can see.  The next token sits at position ``computed`` and
        sees keys from ``computed - window + 1`` on.  Returns the number of pages given back."""
        if not self._windowed:
            return 0
        req = self._requests[rid]
        given = 0
        for gi, g in enumerate(self.groups):
            if g.window <= 0:
                continue
            first_needed = computed - g.window + 1
            if first_needed <= 0:
                continue
            upto_page = min(first_needed // self.page_size, len(req.tables[gi]))
            back = []
            for lp in range(req.trimmed[gi], upto_page):
                if req.tables[gi][lp] >= 0:
                    back.append(req.tables[gi][lp])
                    req.tables[gi][lp] = -1
            if back:
                g.allocator.give_back(back)
                given += len(back)
                req.arrays[gi] = None
            req.trimmed[gi] = max(req.trimmed[gi], upto_page)
        return given

    def release(self, rid) -> None:
        """Give back every page and the state slot of a request."""
        req = self._requests.pop(rid)
        for g, t in zip(self.groups, req.tables):
            g.allocator.give_back([b for b in t if b >= 0])
        self._free_slots.append(req.state_slot)

    def live_requests(self) -> list:
        return list(self._requests)

    # ---- prefix sharing (single full-attention group only) ---------------------------------
    def match_prefix(self, rid, tokens: Sequence[int]) -> int:
        """Point a request without pages at cached pages for its longest known prefix; returns
        the number of tokens covered.  A fully cached prompt gives its last page back so that the
        last position is computed and yields logits (tensorline/batch_engine.py:266-280)."""
        if not self.prefix_caching:
            return 0
        req = self._requests[rid]
        table = req.tables[0]
        if table:
            return 0
        alloc, bs, parent = self.groups[0].allocator, self.page_size, None
        for i in range(len(tokens) // bs):
            content = (parent, tuple(tokens[i * bs:(i + 1) * bs]))
            h = page_key(*content)
            blk = alloc.revive(h, content)
            if blk is None:
                break
            table.append(blk)
            req.hashes.append(h)
            parent = h
        if table and len(table) * bs == len(tokens):
            alloc.give_back([table.pop()])
            req.hashes.pop()
        req.arrays[0] = None
        return len(table) * bs

    def publish(self, rid, tokens: Sequence[int], computed: int) -> None:
        """Register the request's full, computed pages under their content hashes
        (tensorline/batch_engine.py:282-290)."""
        if not self.prefix_caching:
            return
        req = self._requests[rid]
        alloc, bs, table = self.groups[0].allocator, self.page_size, req.tables[0]
        while len(req.hashes) < min(computed, len(tokens)) // bs:
            i = len(req.hashes)
            content = (req.hashes[-1] if i else None, tuple(tokens[i * bs:(i + 1) * bs]))
            h = page_key(*content)
            req.hashes.append(h)
            alloc.publish(table[i], h, content)

    # ---- views for the step function -------------------------------------------------------
    def storage(self, entry: int) -> dict[str, torch.Tensor]:
        """The pages of the entry's planes by name (those of the entry whose cache it reads, if it
        has none of its own); empty for an entry that caches nothing."""
        src = self.storage_entry[entry]
        if src is None:
            return {}
        return self.groups[self.group_of_entry[entry]].storage.get(src, {})

    def owns_storage(self, entry: int) -> bool:
        return self.storage_entry[entry] == entry

    # ---- checks ----------------------------------------------------------------------------
    def check(self) -> None:
        """No page lost, held twice without a reference for each holder, or free while held."""
        for gi, g in enumerate(self.groups):
            held: dict[int, int] = {}
            for req in self._requests.values():
                for b in req.tables[gi]:
                    if b >= 0:
                        held[b] = held.get(b, 0) + 1
            g.allocator.check(held)
        slots = [r.state_slot for r in self._requests.values()]
        if len(set(slots)) != len(slots):
            raise AssertionError("a state slot is held twice")
        if sorted(slots + self._free_slots) != list(range(self.max_requests)):
            raise AssertionError("a state slot is lost")
