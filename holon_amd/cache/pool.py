"""A pool of page ids with reference counts. core/holon/core/memory.py:42-123 (`Pool`).

The last page is the null page: never handed out, where block-table entries of nothing point."""
from __future__ import annotations


class OutOfPages(Exception):
    """The pool cannot give the pages asked for; nothing was taken."""


class PagePool:
    def __init__(self, num_pages: int) -> None:
        if num_pages < 2:
            raise ValueError("a pool needs at least one page beside the null page")
        self.num_pages = num_pages
        self.null = num_pages - 1
        self._free = list(range(num_pages - 2, -1, -1))          # a stack: low ids first, freed pages reused first
        self._refs = [0] * num_pages

    @property
    def usable(self) -> int:
        return self.num_pages - 1

    @property
    def free(self) -> int:
        return len(self._free)

    def alloc(self, n: int) -> list[int]:
        if n > len(self._free):
            raise OutOfPages(f"{n} pages asked, {len(self._free)} free of {self.usable}")
        out = [self._free.pop() for _ in range(n)]
        for p in out:
            self._refs[p] = 1
        return out

    def incref(self, page: int) -> None:
        if self._refs[page] < 1:
            raise RuntimeError(f"page {page} is free: nothing to share")
        self._refs[page] += 1

    def decref(self, page: int) -> None:
        if page == self.null or not 0 <= page < self.num_pages or self._refs[page] < 1:
            raise RuntimeError(f"page {page} released twice (or never held)")
        self._refs[page] -= 1
        if self._refs[page] == 0:
            self._free.append(page)

    def refs(self, page: int) -> int:
        return self._refs[page]
