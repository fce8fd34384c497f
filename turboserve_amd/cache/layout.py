"""Which cache each scheduled layer call has, and how calls with equal needs share a pool.

Calls whose mixers need the same pages (same KV heads, key and value widths and window) form a *group*:
one page pool, one block table per request, one device tensor holding every member's keys and
values.  A model whose layers differ (all keys in some, a window in others) has several
groups, each with pages of its own, so a windowed group can give pages back while the request
runs.  Calls that need fixed-size state get a state tensor indexed by the request's slot.
The reference has one pool with the same block ids for every layer
(src/turboserve/engine/core/kv_cache.py:372-400).
"""

from __future__ import annotations

from collections.abc import Sequence
from dataclasses import dataclass

from turboserve_amd.parts.base import CacheNeed, FixedState, PagedKV


@dataclass(frozen=True)
class PageGroup:
    num_kv_heads: int
    head_dim: int
    window: int | None
    entries: tuple[int, ...]  # schedule entries that own a unit in this group (one per unit: an entry may own several)
    value_dim: int | None = None

    @property
    def value_width(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim

    def elements_per_token(self) -> int:
        """Key and value elements one token takes over all members."""
        return len(self.entries) * self.num_kv_heads * (self.head_dim + self.value_width)


@dataclass(frozen=True)
class CacheLayout:
    groups: tuple[PageGroup, ...]
    state_entries: tuple[tuple[int, FixedState], ...]
    #: per schedule entry: ("pages", group, unit) | ("state", index) | ("reads", entry) | None, or,
    #: for an entry whose mixer has several needs, a tuple of such units in the order of the needs
    entry_units: tuple[tuple | None, ...]

    @classmethod
    def from_needs(cls, needs: Sequence[CacheNeed], reads: Sequence[int | None]) -> "CacheLayout":
        """``needs[i]``: what schedule entry ``i`` owns (one need, or a tuple of needs);
        ``reads[i]``: the earlier entry whose cache it reads instead."""
        keys: list[tuple] = []
        members: list[list[int]] = []
        states: list[tuple[int, FixedState]] = []
        units: list[tuple | None] = []

        def unit_of(entry: int, need) -> tuple | None:
            if isinstance(need, PagedKV):
                key = (need.num_kv_heads, need.head_dim, need.window, need.value_width)
                if key not in keys:
                    keys.append(key)
                    members.append([])
                group = keys.index(key)
                members[group].append(entry)
                return ("pages", group, len(members[group]) - 1)
            if isinstance(need, FixedState):
                states.append((entry, need))
                return ("state", len(states) - 1)
            if need is None:
                return None
            raise TypeError(f"schedule entry {entry} declares an unknown cache need {need!r}")

        for entry, need in enumerate(needs):
            if reads[entry] is not None:
                units.append(("reads", reads[entry]))
            elif isinstance(need, (tuple, list)):
                units.append(tuple(unit_of(entry, one) for one in need))
            else:
                units.append(unit_of(entry, need))
        groups = tuple(PageGroup(k[0], k[1], k[2], tuple(m), None if k[3] == k[1] else k[3]) for k, m in zip(keys, members))
        return cls(groups, tuple(states), tuple(units))

    @classmethod
    def from_model(cls, model) -> "CacheLayout":
        return cls.from_needs(model.cache_needs(), [call.cache_of for call in model.plan.schedule])

    def windows(self) -> list[int | None]:
        return [group.window for group in self.groups]

    def bytes_per_page(self, page_size: int, itemsize: int) -> list[int]:
        """Bytes one page of each group takes (keys and values of all members); for one group
        of all layers this is the reference's ``bytes_per_block`` (kv_cache.py:481-494)."""
        return [group.elements_per_token() * page_size * itemsize for group in self.groups]

    def bytes_per_token(self, itemsize: int) -> int:
        return sum(group.elements_per_token() for group in self.groups) * itemsize
