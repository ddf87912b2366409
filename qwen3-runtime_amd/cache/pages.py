"""Host-side page allocator of one cache group.

A pool hands out page numbers ``0 .. num_pages-1``. Freed pages go to the back
of the free list and come out again after the pages freed before them
(reference, for the same first-in-first-out free list:
qwen3_runtime/engine/block_manager.py:40-41,296-311). The pool knows the
holder of every page, so that a page held twice or freed twice is an error at
the moment it happens, not a wrong logit later.
"""

from __future__ import annotations

from collections import deque
from typing import Hashable


class CacheFull(RuntimeError):
    """Not enough free pages (or state slots) for what was asked."""


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages < 1:
            raise ValueError("num_pages must be positive")
        self.num_pages = int(num_pages)
        self._free: deque[int] = deque(range(self.num_pages))
        self._holder: list[Hashable | None] = [None] * self.num_pages

    @property
    def num_free(self) -> int:
        return len(self._free)

    def take(self, holder: Hashable) -> int:
        if not self._free:
            raise CacheFull("no free page")
        page = self._free.popleft()
        if self._holder[page] is not None:
            raise AssertionError(f"page {page} on the free list is held by {self._holder[page]!r}")
        self._holder[page] = holder
        return page

    def give(self, page: int, holder: Hashable) -> None:
        if not 0 <= page < self.num_pages:
            raise ValueError(f"page {page} is outside the pool of {self.num_pages}")
        if self._holder[page] is None:
            raise AssertionError(f"page {page} is freed twice")
        if self._holder[page] != holder:
            raise AssertionError(f"page {page} is held by {self._holder[page]!r}, not {holder!r}")
        self._holder[page] = None
        self._free.append(page)

    def holder_of(self, page: int) -> Hashable | None:
        return self._holder[page]

    def check(self) -> None:
        """Every page is either free once or held once."""
        free = list(self._free)
        if len(set(free)) != len(free):
            raise AssertionError("a page is on the free list twice")
        for page in range(self.num_pages):
            if (self._holder[page] is None) != (page in set(free)):
                raise AssertionError(f"page {page} is both free and held, or neither")
