"""The host side of the cache: page pools, block tables, groups with windows, state slots.
No page is lost, held twice or freed twice, under random orders of requests."""

from __future__ import annotations

import random

import pytest
import torch

from turboserve_amd.cache.allocator import InvalidPageError, OutOfPagesError, PageAllocator
from turboserve_amd.cache.layout import CacheLayout
from turboserve_amd.cache.manager import PAD_PAGE, CacheManager
from turboserve_amd.cache.sizing import MemoryProfileError, size_cache, window_pages_needed
from turboserve_amd.cache.storage import CacheStorage
from turboserve_amd.cache.state_slots import OutOfStateSlotsError, StateSlotPool
from turboserve_amd.config.engine_config import SchedulerConfig
from turboserve_amd.parts.base import FixedState, PagedKV


def test_allocator_states_and_fifo_reuse():
    """tests/unit/test_kv_cache_storage.py:75-127 in the reference."""
    pool = PageAllocator(4, 16)
    pages = pool.allocate_many(3)
    assert pages == [0, 1, 2] and pool.num_free == 1 and pool.num_in_use == 3
    pool.decref(1)
    pool.decref(0)
    pool.check_invariants()
    assert [pool.allocate(), pool.allocate(), pool.allocate()] == [3, 1, 0]  # least recently freed first
    with pytest.raises(OutOfPagesError):
        pool.allocate()
    with pytest.raises(OutOfPagesError):  # all or nothing
        PageAllocator(2, 4).allocate_many(3)
    pool.decref(2)
    with pytest.raises(InvalidPageError, match="double free"):
        pool.decref(2)
    with pytest.raises(InvalidPageError, match="outside the pool"):
        pool.decref(9)
    assert pool.incref(3) == 2 and pool.decref(3) == 1 and pool.refcount(3) == 1  # shared pages are counted
    with pytest.raises(InvalidPageError, match="free"):
        pool.incref(2)
    pool.reset()
    assert pool.num_free == 4
    pool.check_invariants()


def test_a_huge_pool_costs_nothing_until_used_and_invariants_see_a_lost_page():
    """A pool that fills a large device with a tiny model's pages is hundreds of millions of pages
    long: only pages in use take host memory, the order of reuse is the same, and the
    invariant check still finds a page that is neither free nor held, or both."""
    pool = PageAllocator(10**9, 16)
    assert pool.num_free == 10**9 and pool.allocate_many(3) == [0, 1, 2]
    pool.decref(1)
    assert pool.allocate() == 3 and pool.num_in_use == 3 and pool.refcount(10**9 - 1) == 0
    pool.check_invariants()
    small = PageAllocator(3, 4)
    assert small.allocate_many(3) == [0, 1, 2]
    small.decref(0)
    small.decref(2)
    assert [small.allocate(), small.allocate()] == [0, 2]  # once every page has been out: oldest return first
    small._refs.pop(2)  # a page vanishes from the books
    with pytest.raises(RuntimeError, match="lost"):
        small.check_invariants()
    small._refs[2] = 1
    small._returned.append(2)  # a page both held and free
    with pytest.raises(RuntimeError, match="also free"):
        small.check_invariants()


def test_slots_are_page_major_and_pages_come_as_tokens_do():
    """tests/unit/test_block_manager.py:76-101: slot = page * page_size + offset; pages are taken
    portion by portion, not at admission."""
    manager = CacheManager([None], 8, 4, 2)
    held = manager.admit("a")
    assert held.tables == [[]] and manager.pools[0].num_in_use == 0
    assert manager.append("a", 6) == [[0, 1, 2, 3, 4, 5]]
    assert held.tables == [[0, 1]] and held.num_tokens == 6
    manager.admit("b")
    assert manager.append("b", 3) == [[8, 9, 10]]
    assert manager.append("a", 3) == [[6, 7, 12]]  # a's third page is page 3
    assert manager.get("a").tables == [[0, 1, 3]]
    manager.check_invariants()
    manager.free("a")
    assert manager.pools[0].num_in_use == 1 and not manager.has("a")
    with pytest.raises(KeyError):
        manager.free("a")
    with pytest.raises(ValueError, match="already holds"):
        manager.admit("b")
    manager.admit("c")
    assert manager.append("c", 9) == [[p * 4 + o for p in (4, 5, 6) for o in range(4)][:9]]  # FIFO: freed pages come last
    manager.check_invariants()


def test_running_out_of_pages_is_all_or_nothing():
    manager = CacheManager([None, None], [3, 2], 4, 4)
    manager.admit("a")
    assert manager.can_append("a", 8) and not manager.can_append("a", 9)  # the second group holds 8 tokens
    assert manager.pages_short("a", 12) == [0, 1]
    with pytest.raises(OutOfPagesError):
        manager.append("a", 12)
    assert manager.pools[0].num_in_use == 0 and manager.pools[1].num_in_use == 0  # nothing was taken
    manager.append("a", 8)
    assert not manager.can_append("a", 1)
    assert manager.fits_pool(8, 8) and not manager.fits_pool(9, 8)
    assert not manager.can_admit(4, 4)  # no page of group 1 is free
    manager.check_invariants()


def test_window_groups_give_pages_back_while_the_request_runs():
    """Group 0 keeps every key, group 1 a window of 6: pages wholly below the next query's
    window go back to the pool and their table entries become PAD_PAGE."""
    manager = CacheManager([None, 6], [16, 4], 4, 2)
    manager.admit("a")
    manager.append("a", 10)  # positions 0..9
    assert manager.get("a").tables[1] == [0, 1, 2]
    manager.append("a", 1)  # query at 10 sees keys 5..10: page 0 (keys 0..3) is passed
    assert manager.get("a").tables[1][0] == PAD_PAGE and manager.pools[1].num_in_use == 2
    for _ in range(30):
        manager.append("a", 1)
        manager.check_invariants()
    table = manager.get("a").tables[1]
    assert len(table) == 11 and table.count(PAD_PAGE) == 8 and manager.pools[1].num_in_use == 3
    assert len(manager.get("a").tables[0]) == 11 and PAD_PAGE not in manager.get("a").tables[0]
    assert manager.peak_pages(1, 1000, 1) == 3 and manager.peak_pages(0, 1000, 1) == 250
    assert manager.peak_pages(1, 5, 64) == 2  # a short request needs no more than its own pages
    assert manager.fits_pool(10_000, 1) is False and CacheManager([6], 4, 4, 1).fits_pool(10_000, 1)
    manager.free("a")
    assert manager.pools[1].num_in_use == 0 and manager.pools[0].num_in_use == 0
    # A portion larger than the window: its own keys must all stay until it has run.
    manager.admit("b")
    manager.append("b", 3)
    manager.append("b", 9)  # queries 3..11; the first sees keys from 0
    assert PAD_PAGE not in manager.get("b").tables[1]


def test_state_slots():
    pool = StateSlotPool(2)
    a, b = pool.allocate(), pool.allocate()
    assert {a, b} == {0, 1} and pool.num_free == 0
    with pytest.raises(OutOfStateSlotsError):
        pool.allocate()
    pool.free(a)
    with pytest.raises(ValueError):
        pool.free(a)
    assert pool.allocate() == a
    pool.check_invariants()
    manager = CacheManager([None], 8, 4, 1)
    manager.admit("a")
    assert not manager.can_admit(1, 1)  # pages are free, the slot is not
    manager.free("a")
    assert manager.can_admit(1, 1)


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_never_lose_or_share_a_page(seed):
    rng = random.Random(seed)
    windows = [None, rng.choice([5, 8, 16])]
    manager = CacheManager(windows, [rng.randrange(6, 14), rng.randrange(4, 10)], rng.choice([2, 4, 8]), 4)
    live: list[int] = []
    counter = 0
    for _ in range(400):
        action = rng.random()
        if action < 0.25 and len(live) < 4 and manager.can_admit(1, 8):
            manager.admit(counter)
            live.append(counter)
            counter += 1
        elif action < 0.85 and live:
            request = rng.choice(live)
            n = rng.randrange(1, 9)
            before = manager.get(request).num_tokens
            if manager.can_append(request, n):
                slots = manager.append(request, n)
                for g in range(2):
                    table = manager.get(request).tables[g]
                    size = manager.page_size
                    assert slots[g] == [table[p // size] * size + p % size for p in range(before, before + n)]
            else:
                with pytest.raises(OutOfPagesError):
                    manager.append(request, n)
                assert manager.get(request).num_tokens == before
        elif live:
            manager.free(live.pop(rng.randrange(len(live))))
        manager.check_invariants()
        held = [page for entry in manager._requests.values() for page in entry.tables[1] if page != PAD_PAGE]
        assert len(held) == len(set(held))
    for request in live:
        manager.free(request)
    assert all(pool.num_in_use == 0 for pool in manager.pools) and manager.state_slots.num_free == 4


def test_layout_groups_layers_by_their_needs():
    full, window, state = PagedKV(2, 8), PagedKV(2, 8, 16), FixedState((4, 3))
    layout = CacheLayout.from_needs([full, window, None, window, state, None, full], [None, None, None, None, None, 1, None])
    assert [(g.window, g.entries) for g in layout.groups] == [(None, (0, 6)), (16, (1, 3))]
    assert layout.entry_units == (("pages", 0, 0), ("pages", 1, 0), None, ("pages", 1, 1), ("state", 0), ("reads", 1), ("pages", 0, 1))
    assert layout.state_entries == ((4, state),) and layout.windows() == [None, 16]
    # tests/unit/test_kv_cache_storage.py:267-305: 2 layers, pages of 4, 2 heads of 8, 32-bit: 1024 bytes a page.
    two = CacheLayout.from_needs([full, full], [None, None])
    assert two.bytes_per_page(4, 4) == [1024] and two.bytes_per_token(4) == 256


def test_a_layer_may_keep_pages_and_state_and_values_of_another_width():
    """One schedule entry with several needs gets one unit for each, in order; keys and values
    of different widths (or no values at all) are a group of their own and are sized apart."""
    pages, wide, latent, state = PagedKV(2, 8), PagedKV(2, 8, None, 24), PagedKV(1, 16, None, 0), FixedState((3,))
    layout = CacheLayout.from_needs([(pages, state), wide, (state, None, pages), latent, None, (pages, state)],
                                    [None, None, None, None, 0, None])
    assert layout.entry_units == ((("pages", 0, 0), ("state", 0)), ("pages", 1, 0), (("state", 1), None, ("pages", 0, 1)),
                                  ("pages", 2, 0), ("reads", 0), (("pages", 0, 2), ("state", 2)))
    assert [(g.head_dim, g.value_width, g.entries) for g in layout.groups] == [(8, 8, (0, 2, 5)), (8, 24, (1,)), (16, 0, (3,))]
    assert [entry for entry, _ in layout.state_entries] == [0, 2, 5]
    assert layout.bytes_per_page(4, 2) == [3 * 2 * 16 * 4 * 2, 2 * 32 * 4 * 2, 16 * 4 * 2]
    # a value width said explicitly and equal to the keys' is the same group as one left out
    same = CacheLayout.from_needs([PagedKV(2, 8, None, 8), PagedKV(2, 8)], [None, None])
    assert len(same.groups) == 1 and same.groups[0].value_dim is None
    with pytest.raises(TypeError, match="unknown cache need"):
        CacheLayout.from_needs([(pages, "rows")], [None])

    storage = CacheStorage(layout, [5, 6, 7], 4, 2, torch.float32, "cpu")
    first, second = storage.view_of(0)
    assert tuple(first.k.shape) == (5, 2, 4, 8) and tuple(first.v.shape) == (5, 2, 8, 4) and first.group == 0
    assert tuple(second.state.shape) == (3, 3)
    own = storage.view_of(1)
    assert tuple(own.k.shape) == (6, 2, 4, 8) and tuple(own.v.shape) == (6, 2, 24, 4) and own.group == 1
    slot, nothing, again = storage.view_of(2)
    assert nothing is None and tuple(again.k.shape) == (5, 2, 4, 8) and again.k.data_ptr() != first.k.data_ptr()
    assert slot.state.data_ptr() != second.state.data_ptr()
    only_keys = storage.view_of(3)
    assert tuple(only_keys.k.shape) == (7, 1, 4, 16) and only_keys.v.numel() == 0
    borrowed = storage.view_of(4)  # reads entry 0's units, all read-only
    assert not borrowed[0].writable and not borrowed[1].writable and borrowed[0].k.data_ptr() == first.k.data_ptr()
    assert len(storage.views()) == 6
    assert storage.num_bytes() == sum(c * b for c, b in zip([5, 6, 7], layout.bytes_per_page(4, 4))) + 3 * 3 * 3 * 4


def test_sizing():
    layout = CacheLayout.from_needs([PagedKV(2, 8)] * 2, [None, None])
    scheduler = SchedulerConfig(block_size=4, max_num_batched_tokens=8, max_num_seqs=2)
    sizing = size_cache(layout, scheduler, itemsize=4, memory=(10_000, 10_000), gpu_memory_utilization=1.0)
    assert sizing.num_blocks == [9] and sizing.kv_bytes == 9216 and sizing.reason == "memory budget"  # floor(10000 / 1024)
    capped = size_cache(layout, scheduler, itemsize=4, memory=(10**6, 10**6), max_model_len=10)
    assert capped.num_blocks == [6] and capped.reason == "max_model_len cap"  # ceil(10 / 4) * 2 requests
    explicit = size_cache(layout, SchedulerConfig(block_size=4, max_num_batched_tokens=8, num_blocks=5), itemsize=4)
    assert explicit.num_blocks == [5] and explicit.reason == "explicit num_blocks"
    with pytest.raises(MemoryProfileError):
        size_cache(layout, scheduler, itemsize=4, memory=(500, 10_000))
    mixed = CacheLayout.from_needs([PagedKV(2, 8), PagedKV(2, 8, 16)], [None, None])
    both = size_cache(mixed, scheduler, itemsize=4, memory=(10**5, 10**5), gpu_memory_utilization=1.0)
    assert both.num_blocks[1] == window_pages_needed(16, scheduler) == 14
    assert both.num_blocks[0] == (10**5 - 14 * 512) // 512


def test_page_table_mirror_follows_the_list():
    """The int32 mirror of a block table equals the list after appends, after an overwritten
    entry that was reported, and after growth beyond its first capacity."""
    import numpy as np

    from turboserve_amd.cache.page_table import PageTable, table_array

    table = PageTable()
    assert table_array(table).size == 0 and table == []
    for page in range(40):
        table.append(100 + page)
        if page % 7 == 0:
            assert table_array(table).tolist() == list(table)
    table[3] = -1
    table.entry_changed(3)
    table.append(7)
    mirror = table_array(table)
    assert mirror.dtype == np.int32 and mirror.tolist() == list(table) and mirror[3] == -1
    assert table_array([4, 5, 6]).tolist() == [4, 5, 6]


def test_manager_tables_report_released_pages():
    """Pages a window has passed turn into PAD_PAGE in the list and in its int32 mirror."""
    from turboserve_amd.cache.manager import PAD_PAGE, CacheManager
    from turboserve_amd.cache.page_table import table_array

    manager = CacheManager([None, 8], [16, 16], 4, 2)
    held = manager.admit("r")
    for _ in range(10):
        manager.append("r", 3)
        for table in held.tables:
            assert table_array(table).tolist() == list(table)
    assert held.tables[1][0] == PAD_PAGE and PAD_PAGE not in held.tables[0]
    manager.free("r")
    manager.check_invariants()
