"""The batch of one step: host entries in, one packed device buffer out.

A step holds, for each request in it, that request's next tokens — a whole prompt, a portion
of one, or a single decoded token — concatenated without padding.  The reference describes
the same batch with ``AttnMetadata`` (src/turboserve/engine/core/types.py:244-398) built from
Python lists by four ``torch.tensor`` calls (src/turboserve/engine/runtime/worker.py:190-194);
here all integer inputs travel in one int32 buffer and the context keeps the host's copies of
the lengths, so nothing is read back.
"""

from __future__ import annotations

from collections.abc import Hashable, Sequence
from dataclasses import dataclass, field

import numpy as np
import torch

from turboserve_amd.cache.manager import PAD_PAGE
from turboserve_amd.cache.page_table import table_array


#: Rows of one request that the prefill attention kernel handles per wavefront.
PREFILL_BLOCK_ROWS = 16


@dataclass
class StepEntry:
    """One request's share of a step."""

    request: Hashable
    tokens: Sequence[int]  # its next tokens
    start: int  # position of tokens[0] = tokens of the request already in the cache
    tables: Sequence[Sequence[int]]  # per cache group: the request's block table
    slots: Sequence[Sequence[int]]  # per cache group: one slot per token
    state_slot: int = 0
    want: Sequence[int] = ()  # places among `tokens` whose logits are wanted


@dataclass
class StepContext:
    """What parts see of a step.  Device tensors are int32 views into one buffer."""

    num_tokens: int
    num_seqs: int
    token_ids: torch.Tensor  # [T]
    positions: torch.Tensor  # [T] absolute position of each token in its request
    token_seq: torch.Tensor  # [T] index of each token's request in this step
    query_start_loc: torch.Tensor  # [S + 1] row range of each request
    context_lens: torch.Tensor  # [S] tokens of each request in the cache after this step
    state_slots: torch.Tensor  # [S]
    logit_rows: torch.Tensor  # [n] rows whose logits are wanted
    slot_mapping: list[torch.Tensor]  # per group [T]
    block_tables: list[torch.Tensor]  # per group [S, MB], PAD_PAGE beyond a request's pages
    prefill_blocks: torch.Tensor  # [n, 2]: (request index, first row) of every 16 rows of multi-token requests
    # host copies
    query_lens: list[int] = field(default_factory=list)
    context_lens_host: list[int] = field(default_factory=list)
    max_query_len: int = 0
    max_context_len: int = 0
    num_logit_rows: int = 0
    # Requests that bring more than one token come first, single-token (decode) requests last,
    # so a kernel specialised for either kind gets one contiguous range of requests and rows.
    num_prefill_seqs: int = 0
    num_decode_seqs: int = 0
    num_prefill_tokens: int = 0
    max_prefill_context_len: int = 0
    max_decode_context_len: int = 0
    #: In a recorded (graph) step the host lengths above are upper bounds; the true longest
    #: context of the single-token requests is this one-element device tensor.
    max_decode_context_dev: torch.Tensor | None = None


def validate_entries(entries: Sequence[StepEntry], num_groups: int, page_size: int) -> None:
    """Host checks of a step (types.py:335-398, scheduler.py:270-274): every request once,
    at least one token each, one slot per token, tables that cover the context."""
    seen: set[Hashable] = set()
    for entry in entries:
        if entry.request in seen:
            raise ValueError(f"request {entry.request!r} appears twice in one step")
        seen.add(entry.request)
        count = len(entry.tokens)
        if count < 1:
            raise ValueError(f"request {entry.request!r} brings no token")
        if entry.start < 0:
            raise ValueError(f"request {entry.request!r} starts at {entry.start}")
        if len(entry.tables) != num_groups or len(entry.slots) != num_groups:
            raise ValueError(f"request {entry.request!r}: expected tables and slots for {num_groups} cache groups")
        context = entry.start + count
        for group in range(num_groups):
            if len(entry.slots[group]) != count:
                raise ValueError(f"request {entry.request!r}: {len(entry.slots[group])} slots for {count} tokens")
            if len(entry.tables[group]) * page_size < context:
                raise ValueError(
                    f"request {entry.request!r}: block table of {len(entry.tables[group])} pages "
                    f"does not cover {context} tokens"
                )
        for place in entry.want:
            if not 0 <= place < count:
                raise ValueError(f"request {entry.request!r}: wanted place {place} is outside its {count} tokens")


def _flat(lists: Sequence[Sequence[int]], count: int) -> np.ndarray:
    """The lists one after the other as int32 (each converted in one call: a prompt portion is
    thousands of values)."""
    if not lists:
        return np.zeros(0, dtype=np.int32)
    out = np.concatenate([np.asarray(values, dtype=np.int32) for values in lists])
    if out.size != count:
        raise ValueError(f"{out.size} values for {count} tokens")
    return out


def build_context(
    entries: Sequence[StepEntry],
    *,
    num_groups: int,
    page_size: int,
    device: torch.device | str,
    check: bool = True,
) -> StepContext:
    """Pack a step's entries into device tensors with one copy.

    Rows are ordered with multi-token entries first and single-token entries last (the
    reference's scheduler emits prefills before decodes, src/turboserve/engine/core/scheduler.py:637;
    here any order is accepted and arranged).  ``logit_rows`` keeps the order of the entries as
    given and of each entry's ``want``."""
    if check:
        validate_entries(entries, num_groups, page_size)
    given = list(entries)
    entries = [e for e in given if len(e.tokens) > 1] + [e for e in given if len(e.tokens) <= 1]
    num_prefill_seqs = sum(1 for e in given if len(e.tokens) > 1)
    num_seqs = len(entries)
    query_lens = [len(e.tokens) for e in entries]
    context_lens = [e.start + n for e, n in zip(entries, query_lens)]
    num_tokens = sum(query_lens)
    starts = np.zeros(num_seqs + 1, dtype=np.int32)
    np.cumsum(query_lens, out=starts[1:])
    widths = [max((len(e.tables[g]) for e in entries), default=1) or 1 for g in range(num_groups)]
    row_of = {id(e): int(starts[i]) for i, e in enumerate(entries)}
    logit_rows = [row_of[id(e)] + place for e in given for place in e.want]

    # 16-row blocks of the multi-token requests, those that see the most keys first, so the
    # long ones start early and the short ones fill the tail of the launch.
    blocks = [
        (context_lens[i] - query_lens[i] + min(offset + PREFILL_BLOCK_ROWS, query_lens[i]), i, int(starts[i]) + offset)
        for i in range(num_prefill_seqs)
        for offset in range(0, query_lens[i], PREFILL_BLOCK_ROWS)
    ]
    blocks.sort(key=lambda b: -b[0])
    block_array = np.asarray([[b[1], b[2]] for b in blocks], dtype=np.int32).reshape(-1)

    pieces: list[np.ndarray] = [
        _flat([e.tokens for e in entries], num_tokens),
        np.concatenate([np.arange(e.start, e.start + n, dtype=np.int32) for e, n in zip(entries, query_lens)])
        if num_seqs else np.zeros(0, dtype=np.int32),
        np.repeat(np.arange(num_seqs, dtype=np.int32), query_lens),
        starts,
        np.asarray(context_lens, dtype=np.int32),
        np.asarray([e.state_slot for e in entries], dtype=np.int32),
        np.asarray(logit_rows, dtype=np.int32),
        block_array,
    ]
    for g in range(num_groups):
        pieces.append(_flat([e.slots[g] for e in entries], num_tokens))
        table = np.full((num_seqs, widths[g]), PAD_PAGE, dtype=np.int32)
        for i, e in enumerate(entries):
            row = table_array(e.tables[g])
            table[i, : row.size] = row
        pieces.append(table.reshape(-1))
    sizes = [p.size for p in pieces]
    packed = torch.from_numpy(np.concatenate(pieces)).to(device)
    views = list(torch.split(packed, sizes))
    return StepContext(
        num_tokens=num_tokens,
        num_seqs=num_seqs,
        token_ids=views[0],
        positions=views[1],
        token_seq=views[2],
        query_start_loc=views[3],
        context_lens=views[4],
        state_slots=views[5],
        logit_rows=views[6],
        prefill_blocks=views[7].view(-1, 2),
        slot_mapping=[views[8 + 2 * g] for g in range(num_groups)],
        block_tables=[views[9 + 2 * g].view(num_seqs, widths[g]) for g in range(num_groups)],
        query_lens=query_lens,
        context_lens_host=context_lens,
        max_query_len=max(query_lens, default=0),
        max_context_len=max(context_lens, default=0),
        num_logit_rows=len(logit_rows),
        num_prefill_seqs=num_prefill_seqs,
        num_decode_seqs=num_seqs - num_prefill_seqs,
        num_prefill_tokens=int(starts[num_prefill_seqs]),
        max_prefill_context_len=max(context_lens[:num_prefill_seqs], default=0),
        max_decode_context_len=max(context_lens[num_prefill_seqs:], default=0),
    )
