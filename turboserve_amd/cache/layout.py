"""Which cache each scheduled layer call has, and how calls with equal needs share a pool.

Calls whose mixers need the same pages (same KV heads, head size and window) form a *group*:
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
    entries: tuple[int, ...]  # schedule entries that own a unit in this group

    def elements_per_token(self) -> int:
        """Key and value elements one token takes over all members."""
        return 2 * len(self.entries) * self.num_kv_heads * self.head_dim


@dataclass(frozen=True)
class CacheLayout:
    groups: tuple[PageGroup, ...]
    state_entries: tuple[tuple[int, FixedState], ...]
    #: per schedule entry: ("pages", group, unit) | ("state", index) | ("reads", entry) | None
    entry_units: tuple[tuple | None, ...]

    @classmethod
    def from_needs(cls, needs: Sequence[CacheNeed], reads: Sequence[int | None]) -> "CacheLayout":
        """``needs[i]``: what schedule entry ``i`` owns; ``reads[i]``: the earlier entry whose
        cache it reads instead."""
        keys: list[tuple] = []
        members: list[list[int]] = []
        states: list[tuple[int, FixedState]] = []
        units: list[tuple | None] = []
        for entry, need in enumerate(needs):
            if reads[entry] is not None:
                units.append(("reads", reads[entry]))
            elif isinstance(need, PagedKV):
                key = (need.num_kv_heads, need.head_dim, need.window)
                if key not in keys:
                    keys.append(key)
                    members.append([])
                group = keys.index(key)
                units.append(("pages", group, len(members[group])))
                members[group].append(entry)
            elif isinstance(need, FixedState):
                units.append(("state", len(states)))
                states.append((entry, need))
            elif need is None:
                units.append(None)
            else:
                raise TypeError(f"schedule entry {entry} declares an unknown cache need {need!r}")
        groups = tuple(PageGroup(k[0], k[1], k[2], tuple(m)) for k, m in zip(keys, members))
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
