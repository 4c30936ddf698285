"""Who holds which page of one pool.

A page is free, or held by one owner or several (a count per page: a page that two
block tables name goes back when the second lets go).  The lowest free ids are
handed out first, so that what a run allocates does not depend on the history of the
pool; a request that cannot be met changes nothing.  The free ids live in a heap,
the counts in a list: every operation costs the pages it touches, not the pool.
(The reference's allocator, with the same policy over a set that it sorts per call:
miniserve/kv/allocator.py:12-89.)
"""

from __future__ import annotations

import heapq
from collections.abc import Iterable


class OutOfPagesError(RuntimeError):
    """More pages were asked for than are free.  Nothing was handed out."""


class PageAllocator:
    def __init__(self, num_pages: int) -> None:
        if type(num_pages) is not int or num_pages <= 0:
            raise ValueError(f"a pool has a positive whole number of pages, not {num_pages!r}.")
        self.num_pages = num_pages
        self._free = list(range(num_pages))       # a heap; an ascending list is one
        self._owners = [0] * num_pages            # how many hold each page

    # ---- handing out and taking back ----------------------------------------------------
    def allocate(self, count: int) -> list[int]:
        """The ``count`` lowest free pages, each now held once."""

        if type(count) is not int or count < 0:
            raise ValueError(f"the number of pages to allocate is a whole number, not {count!r}.")
        if count > len(self._free):
            raise OutOfPagesError(f"out of pages: {count} asked for, {len(self._free)} of {self.num_pages} free.")
        pages = [heapq.heappop(self._free) for _ in range(count)]
        for page in pages:
            self._owners[page] = 1
        return pages

    def retain(self, pages: Iterable[int]) -> None:
        """One more owner for each of ``pages``, which must be held already."""

        for page in self._held(pages, "retain"):
            self._owners[page] += 1

    def release(self, pages: Iterable[int]) -> None:
        """One owner less for each of ``pages``; a page without owners is free again."""

        for page in self._held(pages, "release"):
            self._owners[page] -= 1
            if self._owners[page] == 0:
                heapq.heappush(self._free, page)

    def _held(self, pages: Iterable[int], verb: str) -> tuple[int, ...]:
        """``pages`` as a tuple, after checking all of them (so that a refused call has done nothing)."""

        pages = tuple(pages)
        for page in pages:
            if type(page) is not int:
                raise TypeError(f"cannot {verb} {page!r}: a page is named by a whole number.")
            if not 0 <= page < self.num_pages:
                raise IndexError(f"cannot {verb} page {page}: the pool has pages 0..{self.num_pages - 1}.")
        if len(set(pages)) != len(pages):
            raise ValueError(f"cannot {verb} {list(pages)}: a page is named twice in one call.")
        unowned = [page for page in pages if self._owners[page] == 0]
        if unowned:
            raise RuntimeError(f"cannot {verb} pages {unowned}: they are free (released twice, or never allocated).")
        return pages

    # ---- reading ------------------------------------------------------------------------
    def free_count(self) -> int:
        return len(self._free)

    def used_count(self) -> int:
        return self.num_pages - len(self._free)

    def refcount(self, page: int) -> int:
        if type(page) is not int or not 0 <= page < self.num_pages:
            raise IndexError(f"the pool has pages 0..{self.num_pages - 1}, not {page!r}.")
        return self._owners[page]

    def free_ids(self) -> tuple[int, ...]:
        return tuple(sorted(self._free))

    def assert_invariants(self) -> None:
        """Every page is either on the free heap once, with no owner, or off it with at
        least one.  Linear in the pool: for tests and for debugging."""

        on_heap = [0] * self.num_pages
        for page in self._free:
            on_heap[page] += 1
        for page, (times, owners) in enumerate(zip(on_heap, self._owners)):
            if owners < 0 or times > 1 or (times == 1) != (owners == 0):
                raise AssertionError(f"page {page}: {times} times on the free heap with {owners} owners.")
