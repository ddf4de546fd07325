"""A pool of page ids with a last-in-first-out free list.

Like the reference's `BlockAllocator` (src/wllm/engine/kv_cache.py:27-54) the
free list starts as 0..n-1 and hands out from its end, so the page freed last is
used again first.  Unlike it, every page records who holds it: handing out a held
page, or freeing a page that is free or held by someone else, is an error rather
than a silent count.  Exhaustion raises `OutOfPages` (the reference raises a
RuntimeError that callers match by its text, kv_cache.py:34-35,
src/wllm/engine/scheduler.py:421-423).
"""
from __future__ import annotations


class OutOfPages(RuntimeError):
    """No free page is left in a pool."""


class PageAccountingError(AssertionError):
    """A page was freed twice, freed by a stranger or found held twice."""


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError(f"a pool needs at least one page, got {num_pages}")
        self.num_pages = num_pages
        self._free = list(range(num_pages))
        self._holder = [None] * num_pages

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self, holder) -> int:
        if holder is None:
            raise ValueError("a page needs a holder")
        if not self._free:
            raise OutOfPages("KV cache out of memory: no free pages left")
        page = self._free.pop()
        if self._holder[page] is not None:
            raise PageAccountingError(f"page {page} is on the free list and held by {self._holder[page]!r}")
        self._holder[page] = holder
        return page

    def free(self, page: int, holder) -> None:
        if not 0 <= page < self.num_pages:
            raise PageAccountingError(f"page {page} does not exist")
        if self._holder[page] is None:
            raise PageAccountingError(f"page {page} is freed twice")
        if self._holder[page] != holder:
            raise PageAccountingError(f"page {page} is held by {self._holder[page]!r}, freed by {holder!r}")
        self._holder[page] = None
        self._free.append(page)

    def holder(self, page: int):
        return self._holder[page]

    def held_pages(self) -> dict:
        return {p: h for p, h in enumerate(self._holder) if h is not None}

    def check(self) -> None:
        """Every page is either free once or held once."""
        free = set(self._free)
        if len(free) != len(self._free):
            raise PageAccountingError("a page is on the free list twice")
        for p in range(self.num_pages):
            if (p in free) == (self._holder[p] is not None):
                raise PageAccountingError(f"page {p} is {'both free and held' if p in free else 'lost'}")
