"""Pages of the cache as integers: who holds which, which are free, which hold a known prefix.

Semantics of the reference's ``BlockAllocator`` (tensorline/paged.py:28-97): reference-counted
pages, a free list kept in least-recently-freed order, and a content index of full pages (a hash
chained over everything before the page) so that a later request with the same prefix takes the
pages back instead of recomputing them.  A cached page stays in the free list and is evicted
when ``allocate`` needs it.  Unlike the reference, a hit compares the tokens too, so a hash
collision cannot hand out wrong keys.
"""
from __future__ import annotations

from collections import OrderedDict
from typing import Iterable, Sequence


def block_hash(parent: int | None, tokens: Iterable[int]) -> int:
    """Hash of a full page: its tokens chained with the hash of the page before it
    (tensorline/paged.py:96-97)."""
    return hash((parent, tuple(tokens)))


class BlockAllocator:
    def __init__(self, num_blocks: int, prefix_caching: bool = True):
        if num_blocks < 0:
            raise ValueError("num_blocks must be >= 0")
        self.num_blocks = num_blocks
        self.prefix_caching = prefix_caching
        self._free: OrderedDict[int, None] = OrderedDict.fromkeys(range(num_blocks))   # least recently freed first
        self._ref = [0] * num_blocks
        self._hash_of: list[int | None] = [None] * num_blocks
        self._content_of: list[tuple | None] = [None] * num_blocks
        self._cached: dict[int, int] = {}            # content hash -> page

    # ---- counts ------------------------------------------------------------------------
    @property
    def num_free(self) -> int:
        """Pages nobody holds, including cached ones that can be evicted."""
        return len(self._free)

    @property
    def num_cached(self) -> int:
        return len(self._cached)

    def refcount(self, blk: int) -> int:
        return self._ref[blk]

    # ---- allocate / free ---------------------------------------------------------------
    def allocate(self, n: int) -> list[int] | None:
        """``n`` pages or none at all (tensorline/paged.py:57-69)."""
        if n > len(self._free):
            return None
        out = []
        for _ in range(n):
            blk, _ = self._free.popitem(last=False)
            h = self._hash_of[blk]
            if h is not None:                        # its cached contents are gone now
                del self._cached[h]
                self._hash_of[blk] = None
                self._content_of[blk] = None
            self._ref[blk] = 1
            out.append(blk)
        return out

    def free(self, blocks: Sequence[int]) -> None:
        """Drop one reference from each page.  The tail of a sequence is the least shareable, so
        pages go back in reverse: tail pages are evicted first (tensorline/paged.py:71-77)."""
        for blk in reversed(list(blocks)):
            if not 0 <= blk < self.num_blocks:
                raise ValueError(f"page {blk} is outside the pool of {self.num_blocks}")
            if self._ref[blk] <= 0:
                raise AssertionError(f"double free of block {blk}")
            self._ref[blk] -= 1
            if self._ref[blk] == 0:
                self._free[blk] = None

    # ---- prefix cache ------------------------------------------------------------------
    def lookup(self, h: int, content: tuple | None = None) -> int | None:
        """Take a reference on the cached page with content hash ``h``, if there is one
        (tensorline/paged.py:79-87).  ``content`` = (parent hash, tokens) guards against collisions."""
        blk = self._cached.get(h) if self.prefix_caching else None
        if blk is None:
            return None
        if content is not None and self._content_of[blk] is not None and self._content_of[blk] != content:
            return None
        if self._ref[blk] == 0:
            del self._free[blk]
        self._ref[blk] += 1
        return blk

    def register(self, blk: int, h: int, content: tuple | None = None) -> None:
        """Publish a fully computed page under its content hash; the first writer wins
        (tensorline/paged.py:89-93)."""
        if self.prefix_caching and h not in self._cached and self._hash_of[blk] is None:
            self._cached[h] = blk
            self._hash_of[blk] = h
            self._content_of[blk] = content

    # ---- checks ------------------------------------------------------------------------
    def check(self, held: dict[int, int] | None = None) -> None:
        """Every page is either free with no holder or held and not in the free list; with
        ``held`` (page -> number of holders) the reference counts must agree."""
        for blk in range(self.num_blocks):
            in_free = blk in self._free
            if self._ref[blk] == 0 and not in_free:
                raise AssertionError(f"page {blk} is lost: no holder and not free")
            if self._ref[blk] > 0 and in_free:
                raise AssertionError(f"page {blk} is held {self._ref[blk]} times and also free")
            if held is not None and held.get(blk, 0) != self._ref[blk]:
                raise AssertionError(f"page {blk}: {held.get(blk, 0)} holders but reference count {self._ref[blk]}")
        for h, blk in self._cached.items():
            if self._hash_of[blk] != h:
                raise AssertionError(f"cache index of page {blk} is inconsistent")
