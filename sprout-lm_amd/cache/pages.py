"""A pool of fixed-size pages with reference counts (reference: src/kv-cache.ts:94-95, :125-145)."""
from __future__ import annotations


class PageError(RuntimeError):
    pass


class PagePool:
    """Page ids 0..num_pages-1.  Freed pages are handed out again last-in first-out; page 0 first."""

    def __init__(self, num_pages: int):
        if isinstance(num_pages, bool) or not isinstance(num_pages, int) or num_pages <= 0:
            raise ValueError("num_pages must be a positive integer.")
        self.num_pages = num_pages
        self.refs = [0] * num_pages
        self._free = list(range(num_pages - 1, -1, -1))

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self) -> int | None:
        if not self._free:
            return None
        page = self._free.pop()
        self.refs[page] = 1
        return page

    def retain(self, page: int) -> None:
        if self.refs[page] <= 0:
            raise PageError(f"Page {page} is free and cannot be shared.")
        self.refs[page] += 1

    def release(self, page: int) -> None:
        if self.refs[page] <= 0:
            raise PageError(f"Reference count underflow on page {page}.")
        self.refs[page] -= 1
        if self.refs[page] == 0:
            self._free.append(page)
