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
    def __init__(self, num_pages: int, page_size: int) -> None:
        if num_pages < 0:
            raise ValueError(f"num_pages must be non-negative, got {num_pages}")
        if page_size < 1:
            raise ValueError(f"page_size must be positive, got {page_size}")
        self.num_pages = num_pages
        self.page_size = page_size
        self._refs = [0] * num_pages
        self._free: deque[int] = deque(range(num_pages))

    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_in_use(self) -> int:
        return self.num_pages - len(self._free)

    def refcount(self, page: int) -> int:
        self._check_id(page)
        return self._refs[page]

    def allocate(self) -> int:
        """One page with a reference count of 1."""
        if not self._free:
            raise OutOfPagesError(f"no free cache page: {self.num_in_use}/{self.num_pages} in use")
        page = self._free.popleft()
        self._refs[page] = 1
        return page

    def allocate_many(self, count: int) -> list[int]:
        """``count`` pages or none at all (kv_cache.py:211-228)."""
        if count < 0:
            raise ValueError(f"count must be non-negative, got {count}")
        if count > len(self._free):
            raise OutOfPagesError(
                f"cannot allocate {count} pages: {len(self._free)} free, {self.num_in_use}/{self.num_pages} in use"
            )
        return [self.allocate() for _ in range(count)]

    def incref(self, page: int) -> int:
        self._check_id(page)
        if self._refs[page] == 0:
            raise InvalidPageError(f"cannot share page {page}: it is free")
        self._refs[page] += 1
        return self._refs[page]

    def decref(self, page: int) -> int:
        """Drop one reference; at zero the page goes to the back of the free list."""
        self._check_id(page)
        if self._refs[page] == 0:
            raise InvalidPageError(f"double free of page {page}: it is already free")
        self._refs[page] -= 1
        if self._refs[page] == 0:
            self._free.append(page)
        return self._refs[page]

    def decref_many(self, pages: Iterable[int]) -> None:
        for page in pages:
            self.decref(page)

    def reset(self) -> None:
        self._refs = [0] * self.num_pages
        self._free = deque(range(self.num_pages))

    def stats(self) -> dict[str, int]:
        return {"num_pages": self.num_pages, "num_free_pages": self.num_free, "num_pages_in_use": self.num_in_use}

    def check_invariants(self) -> None:
        """Every page is free xor referenced, and no page is on the free list twice (:316-334)."""
        free = set(self._free)
        if len(free) != len(self._free):
            raise PageAllocatorError("a page appears twice on the free list")
        for page, count in enumerate(self._refs):
            if count < 0:
                raise PageAllocatorError(f"page {page} has a negative reference count")
            if count == 0 and page not in free:
                raise PageAllocatorError(f"page {page} is unreferenced but not free (lost)")
            if count > 0 and page in free:
                raise PageAllocatorError(f"page {page} is referenced but also free")

    def _check_id(self, page: int) -> None:
        if not 0 <= page < self.num_pages:
            raise InvalidPageError(f"page id {page} is outside the pool of {self.num_pages}")
