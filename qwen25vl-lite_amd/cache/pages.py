"""A pool of page ids with reference counts (reference src/qwen25vl_lite/cache.py:36-91).

Pages are handed out from a free list (last freed, first reused) and carry a count of their
holders: a request's block table, a second request that adopted a shared prefix, the prefix
cache.  Giving back is strict: an id outside the pool, a page that is already free, or one
count too many is an error, never a silent repair.
"""

from __future__ import annotations

from typing import Dict, List, Sequence

__all__ = ["OutOfPages", "PagePool"]


class OutOfPages(MemoryError):
    """The pool cannot hand out as many pages as were asked for."""


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError("num_pages must be positive")
        self.num_pages = int(num_pages)
        self._free: List[int] = list(range(self.num_pages - 1, -1, -1))  # page 0 goes out first
        self._refs: List[int] = [0] * self.num_pages

    @property
    def num_free(self) -> int:
        return len(self._free)

    def in_use(self) -> int:
        return self.num_pages - len(self._free)

    def refcount(self, page: int) -> int:
        return self._refs[page]

    def allocate(self, n: int = 1) -> List[int]:
        if n < 0:
            raise ValueError("cannot allocate a negative number of pages")
        if n > len(self._free):
            raise OutOfPages(f"cannot allocate {n} pages; only {len(self._free)} free")
        out = [self._free.pop() for _ in range(n)]
        for p in out:
            self._refs[p] = 1
        return out

    def fork(self, pages: Sequence[int]) -> None:
        """One more holder for each page (it must be held already)."""
        for p in pages:
            p = int(p)
            if not 0 <= p < self.num_pages:
                raise ValueError(f"page id {p} is outside [0, {self.num_pages})")
            if self._refs[p] <= 0:
                raise ValueError(f"page {p} is free; a free page cannot be shared")
        for p in pages:
            self._refs[int(p)] += 1

    def free(self, pages: Sequence[int]) -> None:
        """One holder fewer for each page; a page without holders returns to the free list."""
        for p in pages:
            p = int(p)
            if not 0 <= p < self.num_pages:
                raise ValueError(f"page id {p} is outside [0, {self.num_pages})")
            if self._refs[p] <= 0:
                raise ValueError(f"page {p} is already free (double free)")
            self._refs[p] -= 1
            if self._refs[p] == 0:
                self._free.append(p)

    def check(self, holders: Dict[int, int]) -> None:
        """Assert that ``holders`` (page -> number of holders) is exactly what the pool has."""
        free = set(self._free)
        if len(free) != len(self._free):
            raise AssertionError("a page is on the free list twice")
        for p in range(self.num_pages):
            want = holders.get(p, 0)
            if self._refs[p] != want:
                raise AssertionError(f"page {p}: pool counts {self._refs[p]} holders, {want} found")
            if (p in free) != (want == 0):
                raise AssertionError(f"page {p}: on the free list = {p in free}, holders = {want}")
