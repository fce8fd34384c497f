"""Continuous batching with chunked prefill and recompute preemption
(src/turboserve/engine/core/scheduler.py:416-871), first come first served.

Each ``schedule()`` assembles one step under two budgets (tokens, requests):

1. running requests first, in admission order: each gets its next portion of prompt or its
   one decode token (scheduler.py:648-670);
2. then preempted requests, ahead of
3. new arrivals, head of line only: a request that cannot be funded blocks the ones behind it
   (scheduler.py:672-711).

When pages run out for a running request, the most recently admitted running request that is
not already in this step is preempted: its pages and state slot are given back, its computed
count returns to zero, its produced tokens are kept, and it is re-run later as one long
prompt (scheduler.py:748-802).  If nobody else can be preempted the requester itself is.  A
request that could not fit the pool even alone (it grew past it) is finished with reason
``length`` instead of waiting forever; the reference would loop on it.
"""

from __future__ import annotations

import time
from collections import deque
from collections.abc import Sequence as SequenceABC
from dataclasses import dataclass, field

from turboserve_amd.cache.manager import CacheManager
from turboserve_amd.config.engine_config import SchedulerConfig
from turboserve_amd.engine.batch import StepEntry
from turboserve_amd.engine.sequence import Sequence, SeqStatus
from turboserve_amd.sampling.params import FinishReason, SamplingParams


@dataclass
class ScheduledSeq:
    """One request's share of the step being built (scheduler.py:75-164)."""

    seq: Sequence
    num_new_tokens: int
    start: int
    token_ids: list[int]
    slots: list[list[int]]
    tables: list[list[int]]  # the cache manager's own tables, not copies: read before the next scheduling call
    state_slot: int
    is_prefill: bool
    is_chunk: bool  # a portion that does not reach the end of the prompt: no logits, no token

    @property
    def context_len(self) -> int:
        return self.start + self.num_new_tokens

    @property
    def samples(self) -> bool:
        return not self.is_chunk


@dataclass
class SchedulerOutput:
    """A step: portions of prompts first, then decode tokens (scheduler.py:167-288, 637)."""

    scheduled: list[ScheduledSeq] = field(default_factory=list)
    preempted: list[Sequence] = field(default_factory=list)
    dropped: list[Sequence] = field(default_factory=list)  # finished because the pool cannot hold them
    fresh_state_slots: list[int] = field(default_factory=list)
    num_prefill_seqs: int = 0
    num_decode_seqs: int = 0
    num_prefill_tokens: int = 0
    num_decode_tokens: int = 0

    @property
    def is_empty(self) -> bool:
        return not self.scheduled

    @property
    def num_tokens(self) -> int:
        return self.num_prefill_tokens + self.num_decode_tokens

    def sampled(self) -> list[ScheduledSeq]:
        return [item for item in self.scheduled if item.samples]

    def sample_indices(self) -> list[int]:
        """Row of the last token of every request that samples (scheduler.py:216-229)."""
        rows, offset = [], 0
        for item in self.scheduled:
            offset += item.num_new_tokens
            if item.samples:
                rows.append(offset - 1)
        return rows

    def entries(self) -> list[StepEntry]:
        return [
            StepEntry(
                request=item.seq.seq_id,
                tokens=item.token_ids,
                start=item.start,
                tables=item.tables,
                slots=item.slots,
                state_slot=item.state_slot,
                want=[item.num_new_tokens - 1] if item.samples else [],
            )
            for item in self.scheduled
        ]


class Scheduler:
    def __init__(self, config: SchedulerConfig, cache: CacheManager) -> None:
        if cache.page_size != config.block_size:
            raise ValueError(f"the cache has pages of {cache.page_size} tokens, the scheduler expects {config.block_size}")
        self.config = config
        self.cache = cache
        self._waiting: deque[Sequence] = deque()
        self._preempted: deque[Sequence] = deque()
        self._running: list[Sequence] = []
        self._by_request: dict[str, Sequence] = {}
        self._next_seq_id = 0
        self._num_finished = 0
        self._num_admitted = 0
        self._num_preemptions = 0
        self._num_steps = 0
        self._num_prefill_tokens = 0
        self._num_decode_tokens = 0

    # -- arrivals -------------------------------------------------------------------------------

    def add_request(
        self,
        request_id: str,
        prompt_token_ids: SequenceABC[int],
        sampling: SamplingParams | None = None,
        *,
        priority: int = 0,
        arrival: float | None = None,
        sample_seed: int = 0,
    ) -> Sequence:
        """Queue a request (scheduler.py:496-551).  Refused: a duplicate id, an empty prompt, a
        prompt the pool could not hold even alone, and, with chunking off, a prompt longer than
        the token budget."""
        if request_id in self._by_request:
            raise ValueError(f"request id {request_id!r} is already in flight")
        tokens = [int(t) for t in prompt_token_ids]
        if not tokens:
            raise ValueError(f"request {request_id!r} has an empty prompt")
        portion = self.config.max_num_batched_tokens
        if not self.cache.fits_pool(len(tokens), portion):
            need = [self.cache.peak_pages(g, len(tokens), portion) for g in range(self.cache.num_groups)]
            have = [pool.num_pages for pool in self.cache.pools]
            raise ValueError(f"request {request_id!r} needs {need} cache pages but the pools hold {have}")
        if not self.config.enable_chunked_prefill and len(tokens) > portion:
            raise ValueError(
                f"request {request_id!r} has {len(tokens)} prompt tokens, more than max_num_batched_tokens "
                f"({portion}), and chunked prefill is off"
            )
        seq = Sequence(
            seq_id=self._next_seq_id, request_id=request_id, prompt_token_ids=tokens,
            sampling=sampling or SamplingParams(), priority=priority, sample_seed=sample_seed,
        )
        self._next_seq_id += 1
        seq.timing.t_arrival = time.perf_counter() if arrival is None else arrival
        self._by_request[request_id] = seq
        self._waiting.append(seq)
        return seq

    # -- departures -----------------------------------------------------------------------------

    def finish(self, seq: Sequence, reason: FinishReason, *, now: float | None = None, stop_token_id: int | None = None) -> None:
        """Mark finished, give pages and slot back, leave every queue (scheduler.py:553-565)."""
        if seq.is_finished:
            return
        if self.cache.has(seq.seq_id):
            self.cache.free(seq.seq_id)
        self._detach(seq)
        seq.finish(reason, now=now, stop_token_id=stop_token_id)
        self._num_finished += 1

    def abort(self, request_id: str, *, now: float | None = None) -> bool:
        seq = self._by_request.get(request_id)
        if seq is None:
            return False
        self.finish(seq, FinishReason.ABORT, now=now)
        return True

    def append_token(
        self, seq: Sequence, token_id: int, *, eos_token_ids=frozenset(), logprob: float | None = None,
        now: float | None = None,
    ) -> FinishReason | None:
        """Record a sampled token and finish the request if it ends it (scheduler.py:575-594)."""
        seq.append_token(token_id, logprob=logprob, now=now)
        reason = seq.check_stop(token_id, eos_token_ids=eos_token_ids)
        if reason is not None:
            stop = token_id if reason is FinishReason.STOP else None
            self.finish(seq, reason, now=now, stop_token_id=stop)
        return reason

    def resolve_token(
        self, seq: Sequence, place: int, token_id: int, *, eos_token_ids=frozenset(), logprob: float | None = None,
        now: float | None = None,
    ) -> FinishReason | None:
        """``append_token`` for a token whose place was taken ahead of its value
        (``Sequence.append_unread_token``)."""
        seq.set_unread_token(place, token_id, logprob=logprob, now=now)
        reason = seq.check_stop(token_id, eos_token_ids=eos_token_ids)
        if reason is not None:
            stop = token_id if reason is FinishReason.STOP else None
            self.finish(seq, reason, now=now, stop_token_id=stop)
        return reason

    def only_running(self, sequences: SequenceABC[Sequence]) -> bool:
        """Whether ``sequences`` are exactly the requests that could be in the next step: nothing
        waits, nothing is preempted, and the running requests are these."""
        if self._waiting or self._preempted or len(self._running) != len(sequences):
            return False
        running = {seq.seq_id for seq in self._running}
        return all(seq.seq_id in running and seq.status is SeqStatus.RUNNING for seq in sequences)

    def has_unfinished(self) -> bool:
        return bool(self._by_request)

    @property
    def num_unfinished(self) -> int:
        return len(self._by_request)

    def get(self, request_id: str) -> Sequence | None:
        return self._by_request.get(request_id)

    def reset(self) -> None:
        self._waiting.clear()
        self._preempted.clear()
        self._running.clear()
        self._by_request.clear()
        self.cache.reset()

    # -- the step -------------------------------------------------------------------------------

    def schedule(self, *, now: float | None = None) -> SchedulerOutput:
        timestamp = time.perf_counter() if now is None else now
        out = SchedulerOutput()
        budget = [self.config.max_num_batched_tokens, self.config.max_num_seqs]
        scheduled_ids: set[int] = set()
        preempted_now: set[int] = set()
        prefills: list[ScheduledSeq] = []
        decodes: list[ScheduledSeq] = []

        for seq in list(self._running):
            if budget[0] <= 0 or budget[1] <= 0:
                break
            if seq.status is not SeqStatus.RUNNING:
                continue  # preempted a moment ago as somebody's victim
            num_new = seq.num_new_tokens_to_compute(budget[0])
            if num_new <= 0:
                continue
            if not self.config.enable_chunked_prefill and num_new < seq.num_uncomputed_tokens:
                continue
            if not self._make_room(seq, num_new, scheduled_ids, out, preempted_now):
                continue
            self._emit(seq, num_new, budget, scheduled_ids, prefills, decodes, out, checked=True)

        while budget[0] > 0 and budget[1] > 0:
            from_preempted = bool(self._preempted)
            seq = self._preempted[0] if from_preempted else (self._waiting[0] if self._waiting else None)
            if seq is None or seq.seq_id in preempted_now:
                break
            portion = self.config.max_num_batched_tokens
            if not self.cache.fits_pool(seq.num_tokens, portion):
                # It grew past what the pool can hold even alone: end it rather than wait forever.
                self.finish(seq, FinishReason.LENGTH, now=timestamp)
                out.dropped.append(seq)
                continue
            if not self.cache.can_admit(seq.num_tokens, portion):
                break  # head of line: nobody jumps a request that cannot be funded yet
            num_new = seq.num_new_tokens_to_compute(budget[0])
            if num_new <= 0 or (not self.config.enable_chunked_prefill and num_new < seq.num_uncomputed_tokens):
                break
            held = self.cache.admit(seq.seq_id)
            out.fresh_state_slots.append(held.state_slot)
            (self._preempted if from_preempted else self._waiting).popleft()
            seq.status = SeqStatus.RUNNING
            if seq.timing.t_first_scheduled is None:
                seq.timing.t_first_scheduled = timestamp
            self._running.append(seq)
            self._num_admitted += 1
            self._emit(seq, num_new, budget, scheduled_ids, prefills, decodes, out)

        out.scheduled = [*prefills, *decodes]
        out.num_prefill_seqs = len(prefills)
        out.num_decode_seqs = len(decodes)
        out.num_prefill_tokens = sum(item.num_new_tokens for item in prefills)
        out.num_decode_tokens = sum(item.num_new_tokens for item in decodes)
        self._num_steps += 1
        self._num_prefill_tokens += out.num_prefill_tokens
        self._num_decode_tokens += out.num_decode_tokens
        return out

    def _emit(self, seq, num_new, budget, scheduled_ids, prefills, decodes, out, *, checked: bool = False) -> None:
        """Take the slots of ``num_new`` tokens, record the request in the step and advance its
        computed count at once (scheduler.py:713-744).  ``checked``: room was just made."""
        start = seq.num_computed_tokens
        end = start + num_new
        held = self.cache.get(seq.seq_id)
        slots = self.cache.append(seq.seq_id, num_new, checked=checked)
        is_prefill = start < seq.num_prompt_tokens
        item = ScheduledSeq(
            seq=seq, num_new_tokens=num_new, start=start, token_ids=seq.tokens_in_range(start, end),
            slots=slots, tables=held.tables, state_slot=held.state_slot,
            is_prefill=is_prefill, is_chunk=end < seq.num_tokens,
        )
        seq.advance_computed(num_new)
        budget[0] -= num_new
        budget[1] -= 1
        scheduled_ids.add(seq.seq_id)
        (prefills if is_prefill else decodes).append(item)

    # -- when pages run out ---------------------------------------------------------------------

    def _make_room(self, seq, num_new, scheduled_ids, out, preempted_now) -> bool:
        while not self.cache.can_append(seq.seq_id, num_new):
            victim = self._pick_victim(scheduled_ids, seq)
            if victim is None:
                self._preempt(seq, out, preempted_now)
                return False
            self._preempt(victim, out, preempted_now)
        return True

    def _pick_victim(self, scheduled_ids: set[int], requester: Sequence) -> Sequence | None:
        """Lowest priority, then most recently admitted, never one already in this step
        (scheduler.py:770-785)."""
        candidates = [
            other for other in self._running
            if other is not requester and other.seq_id not in scheduled_ids and other.status is SeqStatus.RUNNING
        ]
        if not candidates:
            return None
        return min(candidates, key=lambda other: (other.priority, -other.seq_id))

    def _preempt(self, seq: Sequence, out: SchedulerOutput, preempted_now: set[int]) -> None:
        self.cache.free(seq.seq_id)
        seq.reset_for_recompute()
        if seq in self._running:
            self._running.remove(seq)
        self._preempted.append(seq)
        preempted_now.add(seq.seq_id)
        out.preempted.append(seq)
        self._num_preemptions += 1

    def _detach(self, seq: Sequence) -> None:
        for queue in (self._running, self._preempted, self._waiting):
            if seq in queue:
                queue.remove(seq)
                break
        self._by_request.pop(seq.request_id, None)

    # -- observability --------------------------------------------------------------------------

    def stats(self) -> dict[str, int | float]:
        out: dict[str, int | float] = {
            "num_waiting": len(self._waiting),
            "num_preempted": len(self._preempted),
            "num_running": len(self._running),
            "num_unfinished": len(self._by_request),
            "num_finished": self._num_finished,
            "num_admitted": self._num_admitted,
            "num_preemptions": self._num_preemptions,
            "num_steps": self._num_steps,
            "num_prefill_tokens": self._num_prefill_tokens,
            "num_decode_tokens": self._num_decode_tokens,
        }
        out.update(self.cache.stats())
        return out

    def check_invariants(self) -> None:
        """Queues, statuses and the pools agree (scheduler.py:840-864)."""
        self.cache.check_invariants()
        seen: set[int] = set()
        for queue, status in ((self._running, SeqStatus.RUNNING), (self._preempted, SeqStatus.PREEMPTED),
                              (self._waiting, SeqStatus.WAITING)):
            for seq in queue:
                if seq.status is not status:
                    raise ValueError(f"{seq.request_id!r} is queued as {status.value} but is {seq.status.value}")
                if status is SeqStatus.RUNNING:
                    if self.cache.get(seq.seq_id).num_tokens != seq.num_computed_tokens:
                        raise ValueError(f"{seq.request_id!r}: the cache and the computed count disagree")
                elif self.cache.has(seq.seq_id):
                    raise ValueError(f"{status.value} {seq.request_id!r} still holds cache")
                seen.add(seq.seq_id)
        if len(seen) != len(self._by_request):
            raise ValueError(f"{len(seen)} requests are queued but {len(self._by_request)} are in flight")
        for seq in self._by_request.values():
            if seq.num_computed_tokens > seq.num_tokens:
                raise ValueError(f"{seq.request_id!r} computed more tokens than it holds")
