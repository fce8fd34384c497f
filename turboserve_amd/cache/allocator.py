"""Reference-counted pool of cache pages.

Counterpart of the reference's ``BlockAllocator`` (src/turboserve/engine/core/kv_cache.py:93-369)
without the prefix-cache recycler: a page is either free (count 0, on the free list) or in use
(count > 0, off it).  The free list is FIFO, so the page freed longest ago is reused first
(:109-111).
"""

from __future__ import annotations

from collections import deque
from collections.abc import Iterable


class PageAllocatorError(RuntimeError):
    """The pool's invariant is broken."""


class OutOfPagesError(PageAllocatorError):
    """No free page is left (kv_cache.py:204-208)."""


class InvalidPageError(PageAllocatorError):
    """A page id outside the pool, or a reference dropped that was never taken (:267-285)."""


class PageAllocator:
    """Pages ``0 .. num_pages - 1``.  Only pages in use cost host memory: pages never handed out
    yet are a range (``_fresh .. num_pages - 1``, which a list of free ids would begin with
    anyway), pages given back wait behind them in a queue, and reference counts are kept for
    pages in use only.  A pool that fills a large device with a small model's pages is millions
    of pages long."""

    def __init__(self, num_pages: int, page_size: int) -> None:
        if num_pages < 0:
            raise ValueError(f"num_pages must be non-negative, got {num_pages}")
        if page_size < 1:
            raise ValueError(f"page_size must be positive, got {page_size}")
        self.num_pages = num_pages
        self.page_size = page_size
        self._refs: dict[int, int] = {}  # page -> count, pages in use only
        self._fresh = 0  # pages from here on have never been handed out
        self._returned: deque[int] = deque()  # pages given back, oldest first

    @property
    def num_free(self) -> int:
        return self.num_pages - len(self._refs)

    @property
    def num_in_use(self) -> int:
        return len(self._refs)

    def refcount(self, page: int) -> int:
        self._check_id(page)
        return self._refs.get(page, 0)

    def allocate(self) -> int:
        """One page with a reference count of 1: the page that has been free longest."""
        if self._fresh < self.num_pages:
            page = self._fresh
            self._fresh += 1
        elif self._returned:
            page = self._returned.popleft()
        else:
            raise OutOfPagesError(f"no free cache page: {self.num_in_use}/{self.num_pages} in use")
        self._refs[page] = 1
        return page

    def allocate_many(self, count: int) -> list[int]:
        """``count`` pages or none at all (kv_cache.py:211-228)."""
        if count < 0:
            raise ValueError(f"count must be non-negative, got {count}")
        if count > self.num_free:
            raise OutOfPagesError(
                f"cannot allocate {count} pages: {self.num_free} free, {self.num_in_use}/{self.num_pages} in use"
            )
        return [self.allocate() for _ in range(count)]

    def incref(self, page: int) -> int:
        self._check_id(page)
        if page not in self._refs:
            raise InvalidPageError(f"cannot share page {page}: it is free")
        self._refs[page] += 1
        return self._refs[page]

    def decref(self, page: int) -> int:
        """Drop one reference; at zero the page goes to the back of the free list."""
        self._check_id(page)
        count = self._refs.get(page, 0)
        if count == 0:
            raise InvalidPageError(f"double free of page {page}: it is already free")
        if count == 1:
            del self._refs[page]
            self._returned.append(page)
            return 0
        self._refs[page] = count - 1
        return count - 1

    def decref_many(self, pages: Iterable[int]) -> None:
        for page in pages:
            self.decref(page)

    def reset(self) -> None:
        self._refs = {}
        self._fresh = 0
        self._returned = deque()

    def stats(self) -> dict[str, int]:
        return {"num_pages": self.num_pages, "num_free_pages": self.num_free, "num_pages_in_use": self.num_in_use}

    def check_invariants(self) -> None:
        """Every page is free xor referenced, and no page is on the free list twice (:316-334)."""
        returned = set(self._returned)
        if len(returned) != len(self._returned):
            raise PageAllocatorError("a page appears twice on the free list")
        if not 0 <= self._fresh <= self.num_pages:
            raise PageAllocatorError(f"{self._fresh} pages handed out of a pool of {self.num_pages}")
        for page in returned:
            if not 0 <= page < self._fresh:
                raise PageAllocatorError(f"page {page} was given back but never handed out")
            if page in self._refs:
                raise PageAllocatorError(f"page {page} is referenced but also free")
        for page, count in self._refs.items():
            if not 0 <= page < self._fresh:
                raise PageAllocatorError(f"page {page} is referenced but was never handed out")
            if count < 1:
                raise PageAllocatorError(f"page {page} has a reference count of {count}")
        if len(returned) + len(self._refs) != self._fresh:
            lost = set(range(self._fresh)) - returned - set(self._refs)
            raise PageAllocatorError(f"pages {sorted(lost)[:8]} are unreferenced but not free (lost)")

    def _check_id(self, page: int) -> None:
        if not 0 <= page < self.num_pages:
            raise InvalidPageError(f"page id {page} is outside the pool of {self.num_pages}")
