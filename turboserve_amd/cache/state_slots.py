"""Slots for per-request state of fixed size.

A request takes one slot when it is admitted and gives it back with its pages.  The slot id
indexes the device tensors of every layer that keeps fixed-size state (none in Qwen2: the
pool is there, and unused).  The reference has no such state
(src/turboserve/engine/core/kv_cache.py:372-386 is its only cache kind).
"""

from __future__ import annotations

from collections import deque


class OutOfStateSlotsError(RuntimeError):
    pass


class StateSlotPool:
    def __init__(self, num_slots: int) -> None:
        if num_slots < 0:
            raise ValueError(f"num_slots must be non-negative, got {num_slots}")
        self.num_slots = num_slots
        self._free: deque[int] = deque(range(num_slots))
        self._held: set[int] = set()

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self) -> int:
        if not self._free:
            raise OutOfStateSlotsError(f"no free state slot: all {self.num_slots} are held")
        slot = self._free.popleft()
        self._held.add(slot)
        return slot

    def free(self, slot: int) -> None:
        if slot not in self._held:
            raise ValueError(f"state slot {slot} is not held")
        self._held.remove(slot)
        self._free.append(slot)

    def reset(self) -> None:
        self._free = deque(range(self.num_slots))
        self._held.clear()

    def check_invariants(self) -> None:
        free = set(self._free)
        if len(free) != len(self._free) or free & self._held or len(free) + len(self._held) != self.num_slots:
            raise RuntimeError("state slots are lost or held twice")
