"""Device side of the cache: the page tensors of every group and the state tensors.

Per group one tensor ``[members, 2, num_pages, kv_heads, page_size * head_dim]`` (keys at index
0, values at 1).  A key page of one head is ``[page_size, head_dim]``; a value page is stored
transposed, ``[head_dim, page_size]``, so that the attention kernels load eight consecutive
keys' values of one head dimension at once.  The reference keeps
``[num_blocks, block_size, kv_heads, head_dim]`` per layer
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
        self.pages = [
            torch.zeros(
                (len(group.entries), 2, count, group.num_kv_heads, page_size * group.head_dim),
                dtype=dtype,
                device=device,
            )
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
        return sum(t.numel() * t.element_size() for t in (*self.pages, *self.states))

    def view_of(self, entry: int, *, writable: bool = True) -> CacheView:
        unit = self.layout.entry_units[entry]
        if unit is None:
            return None
        if unit[0] == "reads":
            return self.view_of(unit[1], writable=False)
        if unit[0] == "pages":
            _, group, member = unit
            tensor = self.pages[group][member]
            spec = self.layout.groups[group]
            pages = tensor.shape[1]
            return PagedKVView(
                k=tensor[0].view(pages, spec.num_kv_heads, self.page_size, spec.head_dim),
                v=tensor[1].view(pages, spec.num_kv_heads, spec.head_dim, self.page_size),
                group=group, block_size=self.page_size,
                window=self.layout.groups[group].window, writable=writable,
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
