"""The batch of one step: host entries in, one packed device buffer out.

A step holds, for each request in it, that request's next tokens — a whole prompt, a portion
of one, or a single decoded token — concatenated without padding.  The reference describes
the same batch with ``AttnMetadata`` (src/turboserve/engine/core/types.py:244-398) built from
Python lists by four ``torch.tensor`` calls (src/turboserve/engine/runtime/worker.py:190-194);
here all integer inputs travel in one int32 buffer and the context keeps the host's copies of
the lengths, so nothing is read back.

There is one description of that buffer (``STEP_FIELDS`` / ``GROUP_FIELDS``, and behind them the
fields a model's parts ask for: ``StepField``), one function that fills it (``pack_step``) and
one that checks what it holds (``check_packed``).  An eager step
packs into a fresh buffer of exactly its shape; a recorded step (``decode_graph``) packs into a
pinned buffer of its bucket's shape, the rows beyond the entries being padding.  A field added
to the tables below therefore reaches both.
"""

from __future__ import annotations

from collections.abc import Callable, Hashable, Sequence
from dataclasses import dataclass, field
from typing import Any

import numpy as np
import torch

from turboserve_amd.cache.manager import PAD_PAGE
from turboserve_amd.cache.page_table import table_array


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


@dataclass(frozen=True)
class StepLimits:
    """What a step's integers are checked against before any kernel sees them: the page pools'
    sizes and windows per cache group, the vocabulary, the number of state slots."""

    num_pages: Sequence[int]
    windows: Sequence[int | None]
    vocab_size: int | None = None
    num_state_slots: int | None = None  # slots 0 .. num_state_slots are valid (the last is the padding row)


# ---------------------------------------------------------------------------------------------
# the packed buffer
# ---------------------------------------------------------------------------------------------

#: Every integer field a step carries to the device, in buffer order: name and length in terms
#: of the step's shape (T tokens, S requests, n wanted rows).
STEP_FIELDS: tuple[tuple[str, Callable[[int, int, int], int]], ...] = (
    ("token_ids", lambda t, s, n: t),
    ("positions", lambda t, s, n: t),          # absolute position of each token in its request
    ("token_seq", lambda t, s, n: t),          # index of each token's request in this step
    ("token_source", lambda t, s, n: t),       # >= 0: the token id is that element of the sampler's last result
    ("query_start_loc", lambda t, s, n: s + 1),
    ("context_lens", lambda t, s, n: s),       # tokens of each request in the cache after this step
    ("state_slots", lambda t, s, n: s),
    ("logit_rows", lambda t, s, n: n),
    ("max_decode_context", lambda t, s, n: 1),  # longest context among the single-token requests
)
#: Per cache group (W: the width of the group's block tables in this step).
GROUP_FIELDS: tuple[tuple[str, Callable[[int, int, int], int]], ...] = (
    ("slot_mapping", lambda t, s, w: t),
    ("block_table", lambda t, s, w: s * w),
)


@dataclass(frozen=True)
class StepField:
    """One more integer field of a step, asked for by a part (``Part.step_fields``): it travels
    in the packed buffer like the engine's own, in eager and in recorded steps, and the part
    finds it as ``ctx.extras[name]``.  ``length(T, S, n)`` is its length in a step of ``T``
    tokens, ``S`` requests and ``n`` wanted rows; ``fill(entries)`` gives its values for the
    step's entries (in row order: multi-token entries first), as many as the entries account
    for; what lies beyond them (the padding rows of a recorded shape) is ``pad``."""

    name: str
    length: Callable[[int, int, int], int]
    fill: Callable[[Sequence["StepEntry"]], Sequence[int]]
    pad: int = 0


def merge_step_fields(fields: Sequence[StepField]) -> tuple[StepField, ...]:
    """The distinct fields of a model's parts, in first-seen order.  Every layer's part of a kind
    asks for the same field, so a kind defines its field once (a module-level object that all
    its instances return); different fields under one name are refused."""
    taken = {name for name, _ in STEP_FIELDS} | {name for name, _ in GROUP_FIELDS}
    merged: dict[str, StepField] = {}
    for one in fields:
        if one.name in taken or any(one.name.startswith(name) and one.name[len(name):].isdigit() for name, _ in GROUP_FIELDS):
            raise ValueError(f"step field {one.name!r} is one of the engine's own")
        if one.name in merged and merged[one.name] != one:
            raise ValueError(f"two parts ask for different step fields named {one.name!r}")
        merged.setdefault(one.name, one)
    return tuple(merged.values())


@dataclass(frozen=True)
class StepLayout:
    """Where each field lies in the packed int32 buffer of a step of one shape."""

    num_tokens: int
    num_seqs: int
    num_logit_rows: int
    widths: tuple[int, ...]
    offsets: dict[str, tuple[int, int]]  # name (group fields: name + group index) -> (start, length)
    total: int
    extra: tuple[StepField, ...] = ()  # the parts' own fields, behind the engine's

    @classmethod
    def make(cls, num_tokens: int, num_seqs: int, num_logit_rows: int, widths: Sequence[int],
             extra: Sequence[StepField] = ()) -> "StepLayout":
        offsets: dict[str, tuple[int, int]] = {}
        cursor = 0

        def take(name: str, length: int) -> None:
            nonlocal cursor
            offsets[name] = (cursor, length)
            cursor += -(-length // 4) * 4  # every field starts on 16 bytes

        for name, length in STEP_FIELDS:
            take(name, length(num_tokens, num_seqs, num_logit_rows))
        for group, width in enumerate(widths):
            for name, length in GROUP_FIELDS:
                take(f"{name}{group}", length(num_tokens, num_seqs, width))
        for one in extra:
            take(one.name, one.length(num_tokens, num_seqs, num_logit_rows))
        return cls(num_tokens, num_seqs, num_logit_rows, tuple(widths), offsets, cursor, tuple(extra))

    def view(self, buffer: Any, name: str) -> Any:
        """The field's slice of ``buffer`` (a numpy array or a tensor of ``total`` int32)."""
        start, length = self.offsets[name]
        return buffer[start:start + length]


def _flat(lists: Sequence[Sequence[int]]) -> np.ndarray:
    """The lists one after the other as int32 (each converted in one call: a prompt portion is
    thousands of values)."""
    if not lists:
        return np.zeros(0, dtype=np.int32)
    if all(len(values) == 1 for values in lists):
        return np.asarray([values[0] for values in lists], dtype=np.int32)
    return np.concatenate([np.asarray(values, dtype=np.int32) for values in lists])


def pack_step(
    data: np.ndarray,
    layout: StepLayout,
    entries: Sequence[StepEntry],
    logit_rows: Sequence[int],
    *,
    pad_state_slot: int = 0,
    token_sources: dict[int, int] | None = None,
    recorded: bool = False,
) -> None:
    """Write a step into ``data`` (int32, ``layout.total`` long).  ``entries`` are in row order.
    Where the layout is larger than the step (a recorded shape: more requests, all of one
    token), the rest is padding: position 0, context 1, no cache write, the padding state
    slot.  ``recorded``: the layout is a recorded step's (a bucket's shape, replayed with any
    data), and block-table entries no request uses are page 0, not ``PAD_PAGE``.
    ``token_sources[i] = j``: entry ``i``'s single token is element ``j`` of a device tensor and
    is patched in on the device."""
    live = len(entries)
    seqs, tokens = layout.num_seqs, layout.num_tokens
    query_lens = [len(e.tokens) for e in entries]
    live_tokens = sum(query_lens)
    if live > seqs or live_tokens + (seqs - live) != tokens:
        raise ValueError(f"{live} requests with {live_tokens} tokens do not fit a step shape of {seqs} requests, {tokens} tokens")
    single = live_tokens == live

    def put(name: str, values, pad) -> None:
        out = layout.view(data, name)
        count = len(values)
        out[:count] = values
        out[count:] = pad

    put("token_ids", _flat([e.tokens for e in entries]), 0)
    if single:
        put("positions", [e.start for e in entries], 0)
    else:
        put("positions", np.concatenate([np.arange(e.start, e.start + n, dtype=np.int32) for e, n in zip(entries, query_lens)])
            if live else [], 0)
    seq_of = layout.view(data, "token_seq")
    starts = layout.view(data, "query_start_loc")
    if single:
        seq_of[:] = np.arange(tokens, dtype=np.int32)
        starts[:] = np.arange(seqs + 1, dtype=np.int32)
    else:
        seq_of[:live_tokens] = np.repeat(np.arange(live, dtype=np.int32), query_lens)
        seq_of[live_tokens:] = np.arange(live, seqs, dtype=np.int32)
        starts[0] = 0
        np.cumsum(query_lens, out=starts[1:live + 1])
        starts[live + 1:] = live_tokens + np.arange(1, seqs - live + 1, dtype=np.int32)
    source = layout.view(data, "token_source")
    source[:] = -1
    if token_sources:
        if not single:
            raise ValueError("only single-token entries can take their token from the device")
        source[list(token_sources)] = list(token_sources.values())
    put("context_lens", [e.start + n for e, n in zip(entries, query_lens)], 1)
    put("state_slots", [e.state_slot for e in entries], pad_state_slot)
    put("logit_rows", list(logit_rows), 0)
    layout.view(data, "max_decode_context")[0] = max((e.start + 1 for e in entries if len(e.tokens) == 1), default=1)
    for group, width in enumerate(layout.widths):
        put(f"slot_mapping{group}", _flat([e.slots[group] for e in entries]), -1)  # padding writes nothing
        table = layout.view(data, f"block_table{group}").reshape(seqs, width)
        # Unused entries: PAD_PAGE in an eager step (as the reference pads, types.py:213-234);
        # page 0 in a recorded shape (its rows of padding included), whose kernels may form
        # addresses from a whole row (never read past the context).
        table[:] = 0 if recorded else PAD_PAGE
        for i, e in enumerate(entries):
            row = table_array(e.tables[group])
            table[i, : row.size] = row
    for one in layout.extra:
        values = np.asarray(one.fill(entries), dtype=np.int32).reshape(-1)
        if values.size > layout.offsets[one.name][1]:
            raise ValueError(f"step field {one.name!r}: {values.size} values for a field of {layout.offsets[one.name][1]}")
        put(one.name, values, one.pad)


def check_packed(data: np.ndarray, layout: StepLayout, entries: Sequence[StepEntry], page_size: int,
                 limits: StepLimits) -> None:
    """Refuse, on the host, every integer of a packed step that a kernel would turn into a wild
    address (types.py:335-398 and src/turboserve/engine/model/attention.py:105-112 in the
    reference): a page id outside its pool; ``PAD_PAGE`` inside the range of pages a request's
    queries read (all of them, or from the window's lower bound on); a slot that is neither the
    skip mark nor the place its block table gives the token's position; a token id outside the
    vocabulary; a state slot outside the pool."""
    live = len(entries)
    if live == 0:
        return
    seqs = layout.num_seqs

    def name_of(row: int) -> str:
        return repr(entries[row].request) if row < live else "<padding>"

    starts = layout.view(data, "query_start_loc")
    contexts = layout.view(data, "context_lens").astype(np.int64)
    first_position = contexts - np.diff(starts)  # position of each request's first token in this step
    positions = layout.view(data, "positions").astype(np.int64)
    seq_of = layout.view(data, "token_seq")
    if limits.vocab_size is not None:
        ids = layout.view(data, "token_ids")
        known = layout.view(data, "token_source") < 0
        bad = np.flatnonzero(known & ((ids < 0) | (ids >= limits.vocab_size)))
        if bad.size:
            raise ValueError(f"request {name_of(int(seq_of[bad[0]]))}: token id {int(ids[bad[0]])} is outside "
                             f"the vocabulary of {limits.vocab_size}")
    if limits.num_state_slots is not None:
        slots = layout.view(data, "state_slots")
        bad = np.flatnonzero((slots < 0) | (slots > limits.num_state_slots))
        if bad.size:
            raise ValueError(f"request {name_of(int(bad[0]))}: state slot {int(slots[bad[0]])} is outside "
                             f"the {limits.num_state_slots} slots")
    for group, width in enumerate(layout.widths):
        pool = int(limits.num_pages[group])
        window = limits.windows[group]
        table = layout.view(data, f"block_table{group}").reshape(seqs, width)
        beyond = np.argwhere((table < PAD_PAGE) | (table >= pool))
        if beyond.size:
            row, col = (int(v) for v in beyond[0])
            raise ValueError(f"request {name_of(row)}: page id {int(table[row, col])} at index {col} of its block "
                             f"table of group {group} is outside the pool of {pool} pages")
        # Each request's own table against the pages its context needs (whatever the unused
        # entries of the packed row were filled with).
        for row, entry in enumerate(entries):
            if len(entry.tables[group]) * page_size < int(contexts[row]):
                raise ValueError(f"request {name_of(row)}: its block table of group {group} holds "
                                 f"{len(entry.tables[group])} pages, {int(contexts[row])} tokens need "
                                 f"{-(-int(contexts[row]) // page_size)}")
        lowest_key = np.zeros(seqs, dtype=np.int64) if window is None else np.maximum(0, first_position - window + 1)
        columns = np.arange(width, dtype=np.int64)[None, :]
        read = (columns >= (lowest_key // page_size)[:, None]) & (columns < (-(-contexts // page_size))[:, None])
        missing = np.argwhere(read & (table < 0))
        if missing.size:
            row, col = (int(v) for v in missing[0])
            raise ValueError(f"request {name_of(row)}: no page at index {col} of its block table of group {group}, "
                             f"inside the keys {int(lowest_key[row])}..{int(contexts[row]) - 1} that this step reads")
        slots = layout.view(data, f"slot_mapping{group}").astype(np.int64)
        page = table[seq_of, np.minimum(positions // page_size, width - 1)].astype(np.int64)
        expected = page * page_size + positions % page_size
        bad = np.flatnonzero((slots != -1) & ((slots != expected) | (page < 0) | (positions // page_size >= width)))
        if bad.size:
            t = int(bad[0])
            raise ValueError(f"request {name_of(int(seq_of[t]))}: slot {int(slots[t])} of group {group} is not where "
                             f"its block table puts position {int(positions[t])} (page size {page_size}, pool of {pool} pages)")


# ---------------------------------------------------------------------------------------------
# what parts see
# ---------------------------------------------------------------------------------------------


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
    token_source: torch.Tensor | None = None  # [T], see ``STEP_FIELDS``
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
    #: The longest context of the single-token requests as a one-element device tensor.  In a
    #: recorded step the host lengths above are upper bounds (the shape's) and this is the truth.
    max_decode_context_dev: torch.Tensor | None = None
    #: A recorded step: replayed with other data than it was recorded with, so a part may use
    #: nothing about the step but its shape, the fields above and what ``derive`` refuses there.
    recorded: bool = False
    #: The fields the model's parts asked for (``Part.step_fields``), by name: int32 device views.
    extras: dict = field(default_factory=dict)
    _derived: dict = field(default_factory=dict, repr=False)

    def derive(self, key: Hashable, make: Callable[["StepContext"], Any]) -> Any:
        """What a part computes once per step from the host copies and shares between its
        layers (a launch plan, an index tensor made on the host): ``make(ctx)`` at the first
        call with ``key``, the same object afterwards.  Refused in a recorded step, whose host
        copies are bounds and whose device tensors must be fields of the packed buffer."""
        if self.recorded:
            raise RuntimeError(f"{key!r}: a recorded step has no per-step host data to derive from")
        if key not in self._derived:
            self._derived[key] = make(self)
        return self._derived[key]


def context_views(layout: StepLayout, device_ints: torch.Tensor) -> dict[str, Any]:
    """The device-tensor fields of a :class:`StepContext` as views of the packed buffer."""
    seqs = layout.num_seqs
    groups = range(len(layout.widths))
    return dict(
        token_ids=layout.view(device_ints, "token_ids"),
        positions=layout.view(device_ints, "positions"),
        token_seq=layout.view(device_ints, "token_seq"),
        token_source=layout.view(device_ints, "token_source"),
        query_start_loc=layout.view(device_ints, "query_start_loc"),
        context_lens=layout.view(device_ints, "context_lens"),
        state_slots=layout.view(device_ints, "state_slots"),
        logit_rows=layout.view(device_ints, "logit_rows"),
        max_decode_context_dev=layout.view(device_ints, "max_decode_context"),
        slot_mapping=[layout.view(device_ints, f"slot_mapping{g}") for g in groups],
        block_tables=[layout.view(device_ints, f"block_table{g}").view(seqs, layout.widths[g]) for g in groups],
        extras={one.name: layout.view(device_ints, one.name) for one in layout.extra},
    )


def validate_entries(entries: Sequence[StepEntry], num_groups: int, page_size: int) -> None:
    """Host checks of a step's lists (types.py:335-398, scheduler.py:270-274): every request
    once, at least one token each, one slot per token, tables long enough for the context.
    What the lists hold is checked once packed (``check_packed``)."""
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


def build_context(
    entries: Sequence[StepEntry],
    *,
    num_groups: int,
    page_size: int,
    device: torch.device | str,
    check: bool = True,
    limits: StepLimits | None = None,
    extra_fields: Sequence[StepField] = (),
) -> StepContext:
    """Pack a step's entries into device tensors with one copy.

    Rows are ordered with multi-token entries first and single-token entries last (the
    reference's scheduler emits prefills before decodes, src/turboserve/engine/core/scheduler.py:637;
    here any order is accepted and arranged).  ``logit_rows`` keeps the order of the entries as
    given and of each entry's ``want``.  With ``check`` the lists are validated, and with
    ``limits`` also every page id, slot and token id, before anything is copied."""
    if check:
        validate_entries(entries, num_groups, page_size)
    given = list(entries)
    entries = [e for e in given if len(e.tokens) > 1] + [e for e in given if len(e.tokens) <= 1]
    num_prefill_seqs = sum(1 for e in given if len(e.tokens) > 1)
    num_seqs = len(entries)
    query_lens = [len(e.tokens) for e in entries]
    context_lens = [e.start + n for e, n in zip(entries, query_lens)]
    num_tokens = sum(query_lens)
    first_row, row_of = 0, {}
    for e, n in zip(entries, query_lens):
        row_of[id(e)] = first_row
        first_row += n
    logit_rows = [row_of[id(e)] + place for e in given for place in e.want]
    widths = [max((len(e.tables[g]) for e in entries), default=1) or 1 for g in range(num_groups)]
    layout = StepLayout.make(num_tokens, num_seqs, len(logit_rows), widths, extra_fields)
    data = np.empty(layout.total, dtype=np.int32)
    pack_step(data, layout, entries, logit_rows)
    if check and limits is not None:
        check_packed(data, layout, entries, page_size, limits)
    packed = torch.from_numpy(data).to(device)
    num_prefill_tokens = sum(query_lens[:num_prefill_seqs])
    return StepContext(
        num_tokens=num_tokens,
        num_seqs=num_seqs,
        **context_views(layout, packed),
        query_lens=query_lens,
        context_lens_host=context_lens,
        max_query_len=max(query_lens, default=0),
        max_context_len=max(context_lens, default=0),
        num_logit_rows=len(logit_rows),
        num_prefill_seqs=num_prefill_seqs,
        num_decode_seqs=num_seqs - num_prefill_seqs,
        num_prefill_tokens=num_prefill_tokens,
        max_prefill_context_len=max(context_lens[:num_prefill_seqs], default=0),
        max_decode_context_len=max(context_lens[num_prefill_seqs:], default=0),
    )
