"""A pool of fixed-size cache pages with strict accounting.

A page holds PAGE_TOKENS tokens of one sequence for every layer of a group.
The pool hands out page numbers and takes them back; giving back a page that
is free, or one it never owned, is an error, so that a bookkeeping fault
cannot turn into two sequences writing to one page.
"""

from __future__ import annotations

from typing import List

PAGE_TOKENS = 64  # the kernels (csrc/common.h) use the same number


class CacheFull(RuntimeError):
    pass


def pages_for(tokens: int) -> int:
    return -(-tokens // PAGE_TOKENS)


class PagePool:
    def __init__(self, n_pages: int):
        if n_pages <= 0:
            raise ValueError("a page pool needs at least one page")
        self.n_pages = n_pages
        self._free: List[int] = list(range(n_pages - 1, -1, -1))  # pop() hands out page 0 first
        self._held = [False] * n_pages

    @property
    def n_free(self) -> int:
        return len(self._free)

    @property
    def n_held(self) -> int:
        return self.n_pages - len(self._free)

    def alloc(self) -> int:
        if not self._free:
            raise CacheFull(f"all {self.n_pages} cache pages ({self.n_pages * PAGE_TOKENS} tokens) are in use")
        page = self._free.pop()
        if self._held[page]:
            raise AssertionError(f"page {page} was on the free list while held")
        self._held[page] = True
        return page

    def free(self, page: int) -> None:
        if not 0 <= page < self.n_pages:
            raise ValueError(f"page {page} does not belong to this pool of {self.n_pages}")
        if not self._held[page]:
            raise ValueError(f"page {page} is freed twice")
        self._held[page] = False
        self._free.append(page)

    def check(self) -> None:
        """Raise if a page is lost, held twice or free twice."""
        if len(set(self._free)) != len(self._free):
            raise AssertionError("a page is on the free list twice")
        for page in self._free:
            if self._held[page]:
                raise AssertionError(f"page {page} is both free and held")
        if sum(self._held) + len(self._free) != self.n_pages:
            raise AssertionError("a page is lost")
