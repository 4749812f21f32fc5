"""A pool of fixed-size pages: a free stack and reference counts, no storage.

Page 0 comes out first and the page freed last is handed out next (the reference's pool behaves
the same, src/model/kv_cache.cpp:22-56), so that pages are used again at once and a stale page
shows in tests.  Misuse (releasing a free page, retaining one) raises `PageError`.
"""
from __future__ import annotations

from typing import List


class PageError(RuntimeError):
    """A page was released or retained while free, or does not exist."""


class OutOfPages(RuntimeError):
    """Not enough free pages; nothing was changed."""


class PagePool:
    def __init__(self, n_pages: int):
        if n_pages < 1:
            raise ValueError("a page pool needs at least one page")
        self.n_pages = int(n_pages)
        self._free: List[int] = list(range(self.n_pages - 1, -1, -1))    # a stack; its top is the end
        self._refs = [0] * self.n_pages
        self.on_change = None            # called with (page, new reference count) after every retain and release

    @property
    def free_count(self) -> int:
        return len(self._free)

    def ref_count(self, page: int) -> int:
        self._check(page)
        return self._refs[page]

    def _check(self, page):
        if not 0 <= page < self.n_pages:
            raise PageError(f"page {page} does not exist (the pool has {self.n_pages})")

    def allocate(self) -> int:
        if not self._free:
            raise OutOfPages("no free page left")
        page = self._free.pop()
        self._refs[page] = 1
        return page

    def allocate_many(self, count: int) -> List[int]:
        """`count` pages in the order in which `allocate` would hand them out, or `OutOfPages` with nothing changed."""
        if count > len(self._free):
            raise OutOfPages(f"{count} pages wanted, {len(self._free)} free")
        if count <= 0:
            return []
        pages = self._free[-count:][::-1]
        del self._free[-count:]
        refs = self._refs
        for page in pages:
            refs[page] = 1
        return pages

    def retain(self, page: int) -> None:
        self._check(page)
        if self._refs[page] == 0:
            raise PageError(f"page {page} is free and cannot be retained")
        self._refs[page] += 1
        if self.on_change is not None:
            self.on_change(page, self._refs[page])

    def release(self, page: int) -> None:
        self._check(page)
        if self._refs[page] == 0:
            raise PageError(f"page {page} is already free")
        self._refs[page] -= 1
        if self._refs[page] == 0:
            self._free.append(page)
        if self.on_change is not None:
            self.on_change(page, self._refs[page])
