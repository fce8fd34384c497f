"""Device side of the cache: the page tensors of every group and the state tensors.

Per group one tensor of keys ``[members, num_pages, kv_heads, page_size * head_dim]`` and one of
values ``[members, num_pages, kv_heads, value_dim * page_size]`` (``value_dim`` is ``head_dim``
unless the group's mixers asked for another width, or for none).  A key page of one head is
``[page_size, head_dim]``; a value page is stored transposed, ``[value_dim, page_size]``, so
that the attention kernels load eight consecutive keys' values of one head dimension at once.
The reference keeps ``[num_blocks, block_size, kv_heads, head_dim]`` per layer
(src/turboserve/engine/core/kv_cache.py:372-400); the slot contract (``page * page_size +
offset``) is the same.
"""

from __future__ import annotations

from collections.abc import Sequence

import torch

from turboserve_amd.cache.layout import CacheLayout
from turboserve_amd.parts.base import CacheView, FixedStateView, PagedKVView


class CacheStorage:
    def __init__(
        self,
        layout: CacheLayout,
        num_pages: Sequence[int],
        page_size: int,
        num_state_slots: int,
        dtype: torch.dtype,
        device: torch.device | str,
    ) -> None:
        if len(num_pages) != len(layout.groups):
            raise ValueError(f"{len(num_pages)} pool sizes for {len(layout.groups)} groups")
        if any(count * page_size > 2**31 - 1 for count in num_pages):
            raise ValueError(f"pools of {list(num_pages)} pages of {page_size} tokens: slots would not fit 32-bit integers")
        self.layout = layout
        self.page_size = page_size
        self.num_pages = list(num_pages)
        self.dtype = dtype
        self.key_pages = [
            torch.zeros((len(group.entries), count, group.num_kv_heads, page_size * group.head_dim), dtype=dtype, device=device)
            for group, count in zip(layout.groups, num_pages)
        ]
        self.value_pages = [
            torch.zeros((len(group.entries), count, group.num_kv_heads, group.value_width * page_size), dtype=dtype, device=device)
            for group, count in zip(layout.groups, num_pages)
        ]
        # One row more than there are slots: the row padded batch entries point at.
        self.num_state_slots = num_state_slots
        self.pad_state_slot = num_state_slots
        self.states = [
            torch.zeros((num_state_slots + 1, *need.shape), dtype=need.dtype, device=device)
            for _, need in layout.state_entries
        ]

    def num_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.tensors())

    def tensors(self) -> list[torch.Tensor]:
        """Every device tensor of the cache (keys, values, states)."""
        return [*self.key_pages, *self.value_pages, *self.states]

    def view_of(self, entry: int, *, writable: bool = True) -> CacheView:
        """What schedule entry ``entry`` is handed: the view of its unit, a tuple of views for an
        entry with several units, the (read-only) views of the entry it reads, or ``None``."""
        unit = self.layout.entry_units[entry]
        if unit is not None and len(unit) > 0 and unit[0] == "reads":
            return self.view_of(unit[1], writable=False)
        if unit is not None and (len(unit) == 0 or not isinstance(unit[0], str)):
            return tuple(self._unit_view(one, writable) for one in unit)
        return self._unit_view(unit, writable)

    def _unit_view(self, unit: tuple | None, writable: bool) -> CacheView:
        if unit is None:
            return None
        if unit[0] == "pages":
            _, group, member = unit
            spec = self.layout.groups[group]
            pages = self.num_pages[group]
            return PagedKVView(
                k=self.key_pages[group][member].view(pages, spec.num_kv_heads, self.page_size, spec.head_dim),
                v=self.value_pages[group][member].view(pages, spec.num_kv_heads, spec.value_width, self.page_size),
                group=group, block_size=self.page_size, window=spec.window, writable=writable,
            )
        return FixedStateView(state=self.states[unit[1]], writable=writable)

    def views(self) -> list[CacheView]:
        """One view per schedule entry, in order."""
        return [self.view_of(entry) for entry in range(len(self.layout.entry_units))]

    def zero_state_slots(self, slots: Sequence[int]) -> None:
        """Clear the state of freshly taken slots (a request starts from zero state)."""
        if not slots or not self.states:
            return
        index = torch.tensor(list(slots), dtype=torch.long, device=self.states[0].device)
        for state in self.states:
            state.index_fill_(0, index, 0)
