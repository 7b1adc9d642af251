"""Page bookkeeping on the host: the free list of one layer group and the block
tables of the requests.  Pure Python, no device memory.

The reference keeps one pool and one block table for all layers and returns pages
only when a request ends (cwm/fastgen/generate.py:299-306,1016-1029; free set
cwm/fastgen/utils/iset.py:282-323, lowest ids first).  Here every group of layers
with the same retention need has a pool of its own, and a group whose layers read a
window of keys gives a page back as soon as no later query can reach it.
"""

from __future__ import annotations

import heapq
from typing import List, Optional


class OutOfPages(RuntimeError):
    pass


class PageAccountingError(AssertionError):
    """A page was freed twice, held twice or lost: a bug in the caller."""


class PagePool:
    """Free list of `num_pages` pages; the lowest free id is handed out first, so
    that the same trace always gets the same pages."""

    def __init__(self, num_pages: int) -> None:
        if num_pages <= 0:
            raise ValueError("a pool needs at least one page")
        self.num_pages = num_pages
        self._heap: List[int] = list(range(num_pages))
        self._is_free = [True] * num_pages

    @property
    def free_count(self) -> int:
        return len(self._heap)

    def take(self) -> int:
        if not self._heap:
            raise OutOfPages("no free page")
        page = heapq.heappop(self._heap)
        self._is_free[page] = False
        return page

    def give(self, page: int) -> None:
        if not 0 <= page < self.num_pages:
            raise PageAccountingError(f"page {page} is outside the pool of {self.num_pages}")
        if self._is_free[page]:
            raise PageAccountingError(f"page {page} is freed twice")
        self._is_free[page] = True
        heapq.heappush(self._heap, page)

    def is_free(self, page: int) -> bool:
        return self._is_free[page]


class GroupTable:
    """Block table of one request in one group: logical page -> physical page, -1
    where no page is held (not yet reached, or already given back)."""

    __slots__ = ("pages", "first_held")

    def __init__(self) -> None:
        self.pages: List[int] = []
        self.first_held = 0  # every logical page below this index has been given back, pinned ones apart

    def held(self) -> List[int]:
        return [p for p in self.pages if p >= 0]


def first_page_needed(length: int, window: Optional[int], page_size: int) -> int:
    """Lowest logical page that a query at position >= `length` can still read.

    A layer with window W lets the query at position p read keys p-(W-1)..p
    (cwm/model/transformer.py:253-270), so once a request holds `length` tokens no
    later query reads below length - (W - 1).
    """
    if window is None:
        return 0
    return max(0, length - (window - 1)) // page_size


def pages_for(length: int, page_size: int) -> int:
    """Logical pages that positions 0..length-1 span."""
    return (length + page_size - 1) // page_size
