"""A pool of fixed-size pages with reference counts (reference: src/kv-cache.ts:94-95, :125-145)."""
from __future__ import annotations


class PageError(RuntimeError):
    pass


class _RefCounts:
    """Reference counts by page id; pages never handed out count 0 and take no memory."""

    def __init__(self, num_pages: int):
        self._n = num_pages
        self._counts: list[int] = []      # of the pages handed out so far

    def __len__(self) -> int:
        return self._n

    def __getitem__(self, page: int) -> int:
        if not 0 <= page < self._n:
            raise IndexError(f"page {page} is outside the pool of {self._n}")
        return self._counts[page] if page < len(self._counts) else 0

    def __iter__(self):
        yield from self._counts
        for _ in range(self._n - len(self._counts)):
            yield 0


class PagePool:
    """Page ids 0..num_pages-1.  Freed pages are handed out again last-in first-out; page 0 first.

    The pool costs memory for the pages it has handed out at some time, not for the pages it could hand out:
    an absurd `num_pages` is refused by the memory budget, and must not exhaust the host before that."""

    def __init__(self, num_pages: int):
        if isinstance(num_pages, bool) or not isinstance(num_pages, int) or num_pages <= 0:
            raise ValueError("num_pages must be a positive integer.")
        self.num_pages = num_pages
        self.refs = _RefCounts(num_pages)
        self._given_back: list[int] = []     # stack of released pages

    @property
    def num_free(self) -> int:
        return len(self._given_back) + self.num_pages - len(self.refs._counts)

    def free_list(self) -> list[int]:
        """Free pages in the order in which `allocate` will hand them out."""
        return self._given_back[::-1] + list(range(len(self.refs._counts), self.num_pages))

    def allocate(self) -> int | None:
        counts = self.refs._counts
        if self._given_back:
            page = self._given_back.pop()
        elif len(counts) < self.num_pages:
            page = len(counts)
            counts.append(0)
        else:
            return None
        counts[page] = 1
        return page

    def retain(self, page: int) -> None:
        if self.refs[page] <= 0:
            raise PageError(f"Page {page} is free and cannot be shared.")
        self.refs._counts[page] += 1

    def release(self, page: int) -> None:
        if self.refs[page] <= 0:
            raise PageError(f"Reference count underflow on page {page}.")
        counts = self.refs._counts
        counts[page] -= 1
        if counts[page] == 0:
            self._given_back.append(page)
