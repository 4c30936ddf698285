"""Page allocator with reference counts (reference: miniserve/kv/allocator.py:12-89).

Lowest id first, atomic failure, and the conservation invariants checked after
every public call; the free set is a heap instead of a set sorted per call."""

from __future__ import annotations

import heapq
from collections.abc import Sequence


class OutOfPagesError(RuntimeError):
    pass


class PageAllocator:
    def __init__(self, num_pages: int) -> None:
        if not isinstance(num_pages, int) or isinstance(num_pages, bool) or num_pages <= 0:
            raise ValueError("num_pages must be a positive integer.")
        self.num_pages = num_pages
        self._free_heap = list(range(num_pages))
        self._refcounts = [0] * num_pages
        self._free_count = num_pages

    def allocate(self, count: int) -> list[int]:
        """The ``count`` lowest free ids; nothing changes when they do not exist."""

        if not isinstance(count, int) or isinstance(count, bool) or count < 0:
            raise ValueError("Allocation count must be a non-negative integer.")
        if count > self._free_count:
            raise OutOfPagesError(f"OUT_OF_BLOCKS: requested={count}, free={self._free_count}")
        selected = [heapq.heappop(self._free_heap) for _ in range(count)]
        for page in selected:
            self._refcounts[page] = 1
        self._free_count -= count
        self._check_counts()
        return selected

    def retain(self, pages: Sequence[int]) -> None:
        ids = self._validate(pages)
        if any(self._refcounts[page] == 0 for page in ids):
            raise RuntimeError("Cannot retain a free block.")
        for page in ids:
            self._refcounts[page] += 1
        self._check_counts()

    def release(self, pages: Sequence[int]) -> None:
        ids = self._validate(pages)
        if any(self._refcounts[page] == 0 for page in ids):
            raise RuntimeError("Double free or release of a free block.")
        for page in ids:
            self._refcounts[page] -= 1
            if self._refcounts[page] == 0:
                heapq.heappush(self._free_heap, page)
                self._free_count += 1
        self._check_counts()

    def free_count(self) -> int:
        return self._free_count

    def used_count(self) -> int:
        return self.num_pages - self._free_count

    def refcount(self, page: int) -> int:
        self._validate((page,))
        return self._refcounts[page]

    def free_ids(self) -> tuple[int, ...]:
        return tuple(sorted(self._free_heap))

    def snapshot(self) -> dict[str, object]:
        return {"free_ids": list(self.free_ids()), "refcounts": list(self._refcounts)}

    def _check_counts(self) -> None:
        """The cheap part of the invariants, after every public call."""

        if len(self._free_heap) != self._free_count or not 0 <= self._free_count <= self.num_pages:
            raise AssertionError("Free heap and free count disagree.")

    def assert_invariants(self) -> None:
        """The full check (linear in the pool): every page is either free with
        count 0 or held with a positive count, and the total is conserved."""

        self._check_counts()
        held = sum(1 for count in self._refcounts if count > 0)
        if held + self._free_count != self.num_pages:
            raise AssertionError("Page total is not conserved.")
        if any(count < 0 for count in self._refcounts):
            raise AssertionError("Negative page refcount.")
        if len(set(self._free_heap)) != len(self._free_heap):
            raise AssertionError("A page is on the free list twice.")
        if any(self._refcounts[page] != 0 for page in self._free_heap):
            raise AssertionError("Free list and refcount disagree.")

    def _validate(self, pages: Sequence[int]) -> tuple[int, ...]:
        ids = tuple(pages)
        if len(ids) != len(set(ids)):
            raise ValueError("Duplicate block ID in one operation.")
        if any(not isinstance(page, int) or isinstance(page, bool) for page in ids):
            raise TypeError("Block IDs must be integers.")
        if any(page < 0 or page >= self.num_pages for page in ids):
            raise IndexError("Block ID outside allocator.")
        return ids
