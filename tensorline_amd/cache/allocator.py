"""The pages of one cache group as integers: who holds which, which wait to be handed out, and
which still hold a prefix some later request may want.

Behaviour follows the reference's page allocator (tensorline/paged.py:28-97): a page has a count
of holders; a page nobody holds waits in a queue and is handed out oldest-returned first; a page
that was published under the key of its contents keeps that key while it waits, so a request with
the same prefix can take it back out of the queue instead of computing it again, and loses it
only when the page is handed out for something else.  Beyond the reference, a key is checked
against the tokens it stands for, so two prefixes with the same hash never share a page.

The queue is a doubly linked list threaded through two integer arrays (page ``num_pages`` is the
list's sentinel), so taking a page out of the middle of it, which every prefix hit on a waiting
page does, costs the same as taking one from its front.
"""
from __future__ import annotations

from typing import Iterable, Sequence


def page_key(parent: int | None, tokens: Iterable[int]) -> int:
    """Key of a full page: its tokens together with the key of the page before it, so that equal
    keys mean equal prefixes up to and including this page (tensorline/paged.py:96-97)."""
    return hash((parent, tuple(tokens)))


class PagePool:
    def __init__(self, num_pages: int, share_prefixes: bool = True):
        if num_pages < 0:
            raise ValueError("num_pages must be >= 0")
        n = self.num_pages = num_pages
        self.share_prefixes = share_prefixes
        self._holders = [0] * n
        self._waiting = [True] * n                           # in the queue
        self._after = list(range(1, n + 1)) + [0]    # queue order: sentinel -> 0 -> 1 -> ... -> sentinel
        self._before = [n] + list(range(n))
        self._num_waiting = n
        self._label: list[tuple[int, tuple | None] | None] = [None] * n     # (key, contents) of a published page
        self._page_of_key: dict[int, int] = {}

    # ---- the queue -----------------------------------------------------------------------
    def _leave_queue(self, page: int) -> None:
        a, b = self._before[page], self._after[page]
        self._after[a], self._before[b] = b, a
        self._waiting[page] = False
        self._num_waiting -= 1

    def _join_queue(self, page: int) -> None:
        end = self.num_pages
        last = self._before[end]
        self._after[last], self._before[page] = page, last
        self._after[page], self._before[end] = end, page
        self._waiting[page] = True
        self._num_waiting += 1

    # ---- counts --------------------------------------------------------------------------
    @property
    def num_free(self) -> int:
        """Pages nobody holds, those that still carry a published prefix included."""
        return self._num_waiting

    @property
    def num_cached(self) -> int:
        return len(self._page_of_key)

    def holders(self, page: int) -> int:
        return self._holders[page]

    # ---- handing out and taking back -------------------------------------------------------
    def take(self, count: int) -> list[int] | None:
        """``count`` pages for one holder each, or None and no change if fewer are waiting
        (all or nothing, tensorline/paged.py:57-69).  A page handed out forgets what was published in it."""
        if count > self._num_waiting:
            return None
        got = []
        for _ in range(count):
            page = self._after[self.num_pages]               # the one that has waited longest
            self._leave_queue(page)
            label = self._label[page]
            if label is not None:
                del self._page_of_key[label[0]]
                self._label[page] = None
            self._holders[page] = 1
            got.append(page)
        return got

    def give_back(self, pages: Sequence[int]) -> None:
        """One holder less for each page; a page without holders joins the queue.  The pages of a
        request go back last first, so that its tail, which no other request is likely to share,
        is handed out again before its head (tensorline/paged.py:71-77)."""
        for page in reversed(list(pages)):
            if not 0 <= page < self.num_pages:
                raise ValueError(f"page {page} is outside the pool of {self.num_pages}")
            if self._holders[page] <= 0:
                raise AssertionError(f"double free of page {page}")
            self._holders[page] -= 1
            if self._holders[page] == 0:
                self._join_queue(page)

    # ---- shared prefixes -------------------------------------------------------------------
    def revive(self, key: int, contents: tuple | None = None) -> int | None:
        """The page published under ``key``, with one more holder, or None (tensorline/paged.py:79-87).
        ``contents`` = (parent key, tokens): a page published with other contents is no hit."""
        if not self.share_prefixes:
            return None
        page = self._page_of_key.get(key)
        if page is None:
            return None
        known = self._label[page][1]
        if contents is not None and known is not None and known != contents:
            return None
        if self._waiting[page]:
            self._leave_queue(page)
        self._holders[page] += 1
        return page

    def publish(self, page: int, key: int, contents: tuple | None = None) -> None:
        """Make a fully computed page findable under ``key``.  The first page published under a
        key keeps it, and a page keeps its first key (tensorline/paged.py:89-93)."""
        if self.share_prefixes and key not in self._page_of_key and self._label[page] is None:
            self._page_of_key[key] = page
            self._label[page] = (key, contents)

    # ---- checks ----------------------------------------------------------------------------
    def check(self, held: dict[int, int] | None = None) -> None:
        """Every page either waits without a holder or is held and does not wait; the queue holds
        exactly the waiting pages; with ``held`` (page -> number of holders) the counts agree."""
        queued, page, end = [], self._after[self.num_pages], self.num_pages
        while page != end:
            queued.append(page)
            if len(queued) > self.num_pages:
                raise AssertionError("the queue of waiting pages does not end")
            if self._before[self._after[page]] != page:
                raise AssertionError(f"the queue is broken after page {page}")
            page = self._after[page]
        if len(set(queued)) != len(queued) or len(queued) != self._num_waiting:
            raise AssertionError("the queue of waiting pages holds a page twice or miscounts")
        in_queue = set(queued)
        for page in range(self.num_pages):
            if (page in in_queue) != self._waiting[page]:
                raise AssertionError(f"page {page}: queue and flag disagree")
            if self._holders[page] == 0 and page not in in_queue:
                raise AssertionError(f"page {page} is lost: no holder and not free")
            if self._holders[page] > 0 and page in in_queue:
                raise AssertionError(f"page {page} is held {self._holders[page]} times and also free")
            if held is not None and held.get(page, 0) != self._holders[page]:
                raise AssertionError(f"page {page}: {held.get(page, 0)} holders but a count of {self._holders[page]}")
        for key, page in self._page_of_key.items():
            if self._label[page] is None or self._label[page][0] != key:
                raise AssertionError(f"the index of published pages is inconsistent at page {page}")
