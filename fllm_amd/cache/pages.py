"""Page pool: a LIFO free list with a reference count per page
(rust/engine/src/mem/block_allocator.rs:41-118)."""
from __future__ import annotations

from typing import List


class OutOfPages(MemoryError):
    pass


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages < 0:
            raise ValueError("num_pages must be nonnegative")
        self.num_pages = num_pages
        self.refcounts: List[int] = [0] * num_pages
        self._free: List[int] = list(range(num_pages - 1, -1, -1))   # page 0 is handed out first

    @property
    def available(self) -> int:
        return len(self._free)

    def _check(self, page: int) -> int:
        if not isinstance(page, int) or isinstance(page, bool) or not 0 <= page < self.num_pages:
            raise ValueError(f"invalid page id {page!r}; expected an integer in [0, {self.num_pages})")
        return page

    def alloc(self) -> int:
        if not self._free:
            raise OutOfPages("no free cache pages")
        page = self._free.pop()
        self.refcounts[page] = 1
        return page

    def retain(self, page: int) -> None:
        if self.refcounts[self._check(page)] == 0:
            raise ValueError("cannot acquire an unowned page")
        self.refcounts[page] += 1

    def release(self, page: int) -> bool:
        """True when the page went back to the free list."""
        if self.refcounts[self._check(page)] == 0:
            raise ValueError("cannot release an unowned page")
        self.refcounts[page] -= 1
        if self.refcounts[page] == 0:
            self._free.append(page)      # last freed, first reused
            return True
        return False

    def is_free(self, page: int) -> bool:
        return self.refcounts[self._check(page)] == 0
