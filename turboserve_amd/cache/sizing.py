"""How many cache pages to allocate (src/turboserve/engine/runtime/memory.py:172-381).

An explicit page count wins; otherwise the pages fill what is left of the memory budget after
the weights and an estimate of a step's activations; a ``max_model_len`` caps it at what
``max_num_seqs`` requests of that length can use.  Windowed groups never need more than a
window plus one portion per request, so they are sized to that and the rest goes to the
groups that keep every key.
"""

from __future__ import annotations

from dataclasses import asdict, dataclass
from typing import Any

import torch

from turboserve_amd.cache.layout import CacheLayout
from turboserve_amd.cache.manager import ceil_div
from turboserve_amd.config.engine_config import SchedulerConfig


#: Slots are int32 on the device: a pool holds fewer than this many token places.
MAX_SLOTS = 2**31 - 1


class MemoryProfileError(RuntimeError):
    """No room for a single cache page (memory.py:323-329)."""


@dataclass
class CacheSizing:
    num_blocks: list[int]  # per group
    block_size: int
    bytes_per_block: list[int]  # per group
    kv_bytes: int
    num_slots: int
    budget_bytes: int | None
    activation_bytes: int
    reason: str
    total_bytes: int | None = None
    free_bytes: int | None = None

    def to_dict(self) -> dict[str, Any]:
        return asdict(self)


def activation_headroom_bytes(model, scheduler: SchedulerConfig, itemsize: int) -> int:
    """A step's transient tensors at the scheduler's budgets (memory.py:208-242), as the model's
    own parts report them (``DecoderModel.activation_bytes``)."""
    return model.activation_bytes(scheduler.max_num_batched_tokens, scheduler.max_num_seqs, itemsize)


def window_pages_needed(window: int, scheduler: SchedulerConfig) -> int:
    per_request = ceil_div(window - 1 + scheduler.max_num_batched_tokens, scheduler.block_size) + 1
    return per_request * scheduler.max_num_seqs


def size_cache(
    layout: CacheLayout,
    scheduler: SchedulerConfig,
    *,
    itemsize: int,
    activation_bytes: int = 0,
    gpu_memory_utilization: float = 0.9,
    max_model_len: int | None = None,
    device: torch.device | str | None = None,
    memory: tuple[int, int] | None = None,
) -> CacheSizing:
    """``memory`` is ``(free, total)`` bytes; by default it is probed on ``device``
    (``torch.cuda.mem_get_info``, memory.py:183-187)."""
    page = scheduler.block_size
    per_page = layout.bytes_per_page(page, itemsize)
    windows = layout.windows()
    cap = None if max_model_len is None else ceil_div(max_model_len, page) * scheduler.max_num_seqs

    def clamp(group: int, count: int) -> int:
        count = min(count, MAX_SLOTS // page)  # slots (page * page size + offset) travel as int32
        if windows[group] is not None:
            count = min(count, window_pages_needed(windows[group], scheduler))
        if cap is not None:
            count = min(count, cap)
        return count

    if scheduler.num_blocks is not None:
        counts = [clamp(g, scheduler.num_blocks) if windows[g] is not None else scheduler.num_blocks
                  for g in range(len(per_page))]
        return CacheSizing(counts, page, per_page, sum(c * b for c, b in zip(counts, per_page)),
                           min(c * page for c in counts), None, activation_bytes, "explicit num_blocks")
    if memory is None:
        free, total = torch.cuda.mem_get_info(device)
    else:
        free, total = memory
    used = total - free
    budget = int(total * gpu_memory_utilization) - used - activation_bytes
    counts = [0] * len(per_page)
    remaining = budget
    for g, window in enumerate(windows):
        if window is not None:
            counts[g] = clamp(g, window_pages_needed(window, scheduler))
            remaining -= counts[g] * per_page[g]
    full = [g for g, window in enumerate(windows) if window is None]
    if full:
        share = remaining // sum(per_page[g] for g in full)
        for g in full:
            counts[g] = clamp(g, max(0, share))
    if remaining < 0 or any(c < 1 for c in counts):
        raise MemoryProfileError(
            f"no room for a cache page: budget {budget} bytes after {used} used and {activation_bytes} "
            f"for activations; pages take {per_page} bytes"
        )
    reason = "memory budget" if cap is None or any(counts[g] < cap for g in full) else "max_model_len cap"
    return CacheSizing(counts, page, per_page, sum(c * b for c, b in zip(counts, per_page)),
                       min(c * page for c in counts), budget, activation_bytes, reason, total, free)
