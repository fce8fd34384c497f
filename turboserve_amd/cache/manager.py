"""Host side of the cache: who holds which pages and which state slot.

One page pool and one block table per request *for each group* of layers.  A request's pages
are taken portion by portion as its tokens are scheduled (the reference's ``append_slots``,
src/turboserve/engine/core/block_manager.py:222-246) and given back when it finishes, is
preempted, or, in a windowed group, when every later query's window has passed them.  A slot
is ``page * page_size + offset`` (block_manager.py:248-268).  Released entries of a block
table hold ``PAD_PAGE``; no kernel reads below a window's lower bound.
"""

from __future__ import annotations

from collections.abc import Hashable, Sequence
from dataclasses import dataclass, field

from turboserve_amd.cache.allocator import OutOfPagesError, PageAllocator
from turboserve_amd.cache.page_table import PageTable
from turboserve_amd.cache.state_slots import StateSlotPool

#: Fill value of unused block-table entries (src/turboserve/engine/core/types.py:64-65).
PAD_PAGE = -1


def ceil_div(a: int, b: int) -> int:
    return -(-a // b)


@dataclass
class RequestCache:
    """What one request holds."""

    tables: list[list[int]]  # per group, logical page index -> page id or PAD_PAGE
    num_tokens: int = 0  # tokens that have slots
    state_slot: int = -1
    state_is_fresh: bool = True  # the slot has not been zeroed on the device yet
    released: list[int] = field(default_factory=list)  # per group, leading pages given back


class CacheManager:
    def __init__(
        self,
        windows: Sequence[int | None],
        num_pages: Sequence[int] | int,
        page_size: int,
        num_state_slots: int,
    ) -> None:
        if page_size < 1 or page_size & (page_size - 1):
            raise ValueError(f"page_size must be a power of two, got {page_size}")
        counts = [num_pages] * len(windows) if isinstance(num_pages, int) else list(num_pages)
        if len(counts) != len(windows):
            raise ValueError(f"{len(counts)} pool sizes for {len(windows)} groups")
        self.windows = list(windows)
        self.page_size = page_size
        self.pools = [PageAllocator(n, page_size) for n in counts]
        self.state_slots = StateSlotPool(num_state_slots)
        self._requests: dict[Hashable, RequestCache] = {}

    # -- queries ------------------------------------------------------------------------------

    @property
    def num_groups(self) -> int:
        return len(self.pools)

    def has(self, request: Hashable) -> bool:
        return request in self._requests

    def get(self, request: Hashable) -> RequestCache:
        try:
            return self._requests[request]
        except KeyError:
            raise KeyError(f"request {request!r} holds no cache") from None

    def peak_pages(self, group: int, total_tokens: int, max_portion: int) -> int:
        """Most pages of ``group`` a request of ``total_tokens`` holds at once when its
        portions are at most ``max_portion`` tokens: all of them, or what a window plus one
        portion spans (one more for the window's start inside a page)."""
        pages = ceil_div(total_tokens, self.page_size)
        window = self.windows[group]
        if window is None:
            return pages
        return min(pages, ceil_div(window - 1 + max_portion, self.page_size) + 1)

    def fits_pool(self, total_tokens: int, max_portion: int) -> bool:
        """Whether the request could run if it had the pools to itself."""
        return all(
            self.peak_pages(g, total_tokens, max_portion) <= self.pools[g].num_pages
            for g in range(self.num_groups)
        )

    def can_admit(self, total_tokens: int, max_portion: int) -> bool:
        """Free pages cover the request's peak need in every group and a state slot is free
        (block_manager.py:151-164: the whole sequence must fit, though pages are taken as
        portions are scheduled)."""
        if self.state_slots.num_free < 1:
            return False
        return all(
            self.peak_pages(g, total_tokens, max_portion) <= self.pools[g].num_free
            for g in range(self.num_groups)
        )

    # -- a request's life ---------------------------------------------------------------------

    def admit(self, request: Hashable) -> RequestCache:
        if request in self._requests:
            raise ValueError(f"request {request!r} already holds a cache")
        entry = RequestCache(
            tables=[PageTable() for _ in self.pools],
            state_slot=self.state_slots.allocate(),
            released=[0] * len(self.pools),
        )
        self._requests[request] = entry
        return entry

    def _releasable(self, entry: RequestCache, group: int, start: int) -> int:
        """Leading logical pages no query at position ``>= start`` can see."""
        window = self.windows[group]
        if window is None:
            return 0
        lowest_key = max(0, start - window + 1)
        return min(lowest_key // self.page_size, len(entry.tables[group]))

    def pages_short(self, request: Hashable, num_new: int) -> list[int]:
        """Per group, how many pages more than are free a portion of ``num_new`` tokens needs
        (0: it fits), counting pages the portion's own window lets go."""
        entry = self.get(request)
        end = entry.num_tokens + num_new
        short = []
        for g, pool in enumerate(self.pools):
            grow = max(0, ceil_div(end, self.page_size) - len(entry.tables[g]))
            gain = self._releasable(entry, g, entry.num_tokens) - entry.released[g]
            short.append(max(0, grow - pool.num_free - max(0, gain)))
        return short

    def can_append(self, request: Hashable, num_new: int) -> bool:
        return not any(self.pages_short(request, num_new))

    def append(self, request: Hashable, num_new: int, *, checked: bool = False) -> list[list[int]]:
        """Take pages for the request's next ``num_new`` tokens; returns their slots per group.

        Pages a window has passed are given back first.  All-or-nothing over the groups.
        ``checked``: the caller has just seen :meth:`can_append` say yes for the same arguments
        (the scheduler's case, once per request per step), so the check is not repeated."""
        if num_new < 0:
            raise ValueError(f"num_new must be non-negative, got {num_new}")
        entry = self.get(request)
        if not checked and any(self.pages_short(request, num_new)):
            raise OutOfPagesError(f"request {request!r} cannot grow by {num_new} tokens: pages are short")
        start, end = entry.num_tokens, entry.num_tokens + num_new
        slots: list[list[int]] = []
        for g, pool in enumerate(self.pools):
            table = entry.tables[g]
            upto = self._releasable(entry, g, start)
            for index in range(entry.released[g], upto):
                pool.decref(table[index])
                table[index] = PAD_PAGE
                table.entry_changed(index)
            entry.released[g] = max(entry.released[g], upto)
            while len(table) * self.page_size < end:
                table.append(pool.allocate())
            size = self.page_size
            if num_new == 1:  # a decoded token: no loop
                slots.append([table[start // size] * size + start % size])
            else:
                slots.append([table[pos // size] * size + pos % size for pos in range(start, end)])
        entry.num_tokens = end
        return slots

    def free(self, request: Hashable) -> None:
        """Give back everything the request holds (finish, abort, preemption)."""
        entry = self._requests.pop(request, None)
        if entry is None:
            raise KeyError(f"request {request!r} holds no cache")
        for g, pool in enumerate(self.pools):
            pool.decref_many(page for page in entry.tables[g] if page != PAD_PAGE)
        self.state_slots.free(entry.state_slot)

    def reset(self) -> None:
        self._requests.clear()
        for pool in self.pools:
            pool.reset()
        self.state_slots.reset()

    # -- observability ------------------------------------------------------------------------

    @property
    def num_free_pages(self) -> list[int]:
        return [pool.num_free for pool in self.pools]

    def stats(self) -> dict[str, int]:
        out: dict[str, int] = {"num_cached_requests": len(self._requests)}
        for g, pool in enumerate(self.pools):
            for key, value in pool.stats().items():
                out[f"group{g}_{key}"] = value
        out["num_free_state_slots"] = self.state_slots.num_free
        return out

    def check_invariants(self) -> None:
        """No page lost, held twice or free while held; tables cover the tokens."""
        self.state_slots.check_invariants()
        slots = [entry.state_slot for entry in self._requests.values()]
        if len(set(slots)) != len(slots):
            raise RuntimeError("two requests hold the same state slot")
        for g, pool in enumerate(self.pools):
            pool.check_invariants()
            held: dict[int, int] = {}
            for request, entry in self._requests.items():
                table = entry.tables[g]
                if len(table) * self.page_size < entry.num_tokens:
                    raise RuntimeError(f"{request!r}: group {g} table does not cover {entry.num_tokens} tokens")
                for index, page in enumerate(table):
                    if page == PAD_PAGE:
                        if index >= entry.released[g]:
                            raise RuntimeError(f"{request!r}: group {g} page {index} is missing")
                        continue
                    held[page] = held.get(page, 0) + 1
            for page, count in held.items():
                if pool.refcount(page) != count:
                    raise RuntimeError(
                        f"group {g} page {page}: held {count} times, reference count {pool.refcount(page)}"
                    )
            if len(held) != pool.num_in_use:
                raise RuntimeError(f"group {g}: {pool.num_in_use} pages in use but {len(held)} are in tables")
