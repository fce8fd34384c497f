"""One request as the scheduler sees it (src/turboserve/engine/core/sequence.py:51-374).

Progress is one counter: ``num_computed_tokens`` tokens have keys and values in the cache; the
tokens to run next are the uncomputed ones, capped by the step's budget.  A fresh prompt, a
portion of a prompt and a decoding request (exactly one uncomputed token: the one just
sampled) are the same arithmetic (sequence.py:11-16, 231-241).
"""

from __future__ import annotations

import time
from dataclasses import dataclass, field
from enum import Enum

import numpy as np

from turboserve_amd.sampling.params import FinishReason, SamplingParams


class SeqStatus(str, Enum):
    WAITING = "waiting"
    RUNNING = "running"
    PREEMPTED = "preempted"
    FINISHED = "finished"


@dataclass
class RequestTiming:
    """Wall-clock marks of a request (src/turboserve/engine/core/types.py:146-193)."""

    t_arrival: float | None = None
    t_first_scheduled: float | None = None
    t_first_token: float | None = None
    t_finished: float | None = None

    def _span(self, a: float | None, b: float | None) -> float | None:
        return None if a is None or b is None else b - a

    @property
    def queue_time(self) -> float | None:
        return self._span(self.t_arrival, self.t_first_scheduled)

    @property
    def ttft(self) -> float | None:
        return self._span(self.t_arrival, self.t_first_token)

    @property
    def e2e(self) -> float | None:
        return self._span(self.t_arrival, self.t_finished)

    def tpot(self, num_output_tokens: int) -> float | None:
        span = self._span(self.t_first_token, self.t_finished)
        if span is None or num_output_tokens < 2:
            return None
        return span / (num_output_tokens - 1)


@dataclass
class Sequence:
    seq_id: int
    request_id: str
    prompt_token_ids: list[int]
    sampling: SamplingParams
    priority: int = 0
    sample_seed: int = 0
    output_token_ids: list[int] = field(default_factory=list)
    output_logprobs: list[float] = field(default_factory=list)
    num_computed_tokens: int = 0
    status: SeqStatus = SeqStatus.WAITING
    finish_reason: FinishReason | None = None
    stop_token_id: int | None = None
    num_preemptions: int = 0
    timing: RequestTiming = field(default_factory=RequestTiming)
    #: What ``token_array`` keeps between calls: the tokens as int32 and how many output tokens it holds.
    _token_array: "np.ndarray | None" = field(default=None, repr=False, compare=False)
    _array_outputs: int = field(default=0, repr=False, compare=False)

    # -- token accounting -----------------------------------------------------------------------

    @property
    def num_prompt_tokens(self) -> int:
        return len(self.prompt_token_ids)

    @property
    def num_output_tokens(self) -> int:
        return len(self.output_token_ids)

    @property
    def num_tokens(self) -> int:
        return len(self.prompt_token_ids) + len(self.output_token_ids)

    @property
    def num_uncomputed_tokens(self) -> int:
        return self.num_tokens - self.num_computed_tokens

    @property
    def is_finished(self) -> bool:
        return self.status is SeqStatus.FINISHED

    @property
    def token_ids(self) -> list[int]:
        return [*self.prompt_token_ids, *self.output_token_ids]

    def tokens_in_range(self, start: int, end: int) -> list[int]:
        """Tokens ``start..end-1`` of prompt followed by output."""
        n = len(self.prompt_token_ids)
        if end <= n:
            return self.prompt_token_ids[start:end]
        if start >= n:
            return self.output_token_ids[start - n:end - n]
        return [*self.prompt_token_ids[start:], *self.output_token_ids[:end - n]]

    def num_new_tokens_to_compute(self, budget: int) -> int:
        if self.is_finished or budget <= 0:
            return 0
        return max(0, min(budget, self.num_uncomputed_tokens))

    def advance_computed(self, num_tokens: int) -> None:
        if num_tokens < 0 or self.num_computed_tokens + num_tokens > self.num_tokens:
            raise ValueError(
                f"sequence {self.request_id!r} cannot advance by {num_tokens}: "
                f"{self.num_computed_tokens} computed of {self.num_tokens}"
            )
        self.num_computed_tokens += num_tokens

    def token_array(self) -> "np.ndarray":
        """``token_ids`` as an int32 array that is kept and extended from call to call (a request
        with a repetition penalty hands its whole history to the sampler every step: building it
        from the lists costs 30 us per thousand tokens, this a copy of what is new).  The last
        output tokens held may have been stand-ins for unread ones, so they are taken again."""
        prompt, outputs = self.prompt_token_ids, self.output_token_ids
        total = len(prompt) + len(outputs)
        array = self._token_array
        if array is None or array.shape[0] < total:
            grown = np.empty(max(total + 64, 2 * (0 if array is None else array.shape[0])), dtype=np.int32)
            grown[:len(prompt)] = prompt
            self._array_outputs = 0
            array = self._token_array = grown
        first = max(0, min(self._array_outputs, len(outputs)) - 2)
        array[len(prompt) + first:total] = outputs[first:]
        self._array_outputs = len(outputs)
        return array[:total]

    def reset_for_recompute(self) -> None:
        """Forget the cache, keep the output: the tokens already produced are recomputed as if
        they were prompt, not produced again (sequence.py:256-267)."""
        self.num_computed_tokens = 0
        self.num_preemptions += 1
        self.status = SeqStatus.PREEMPTED

    # -- generation -----------------------------------------------------------------------------

    def append_token(self, token_id: int, *, logprob: float | None = None, now: float | None = None) -> None:
        if self.is_finished:
            raise ValueError(f"sequence {self.request_id!r} finished with {self.finish_reason}; no token can be appended")
        self.output_token_ids.append(int(token_id))
        if logprob is not None:
            self.output_logprobs.append(float(logprob))
        if self.timing.t_first_token is None:
            self.timing.t_first_token = time.perf_counter() if now is None else now

    #: Stands in the output for a token that is sampled but has not been read from the device.
    UNREAD_TOKEN = -1

    def append_unread_token(self) -> int:
        """Make room for a token whose value is not known yet (the step after the one that
        samples it is being prepared); returns its place in ``output_token_ids`` for
        ``set_unread_token``."""
        if self.is_finished:
            raise ValueError(f"sequence {self.request_id!r} finished with {self.finish_reason}; no token can be appended")
        self.output_token_ids.append(self.UNREAD_TOKEN)
        return len(self.output_token_ids) - 1

    def set_unread_token(self, place: int, token_id: int, *, logprob: float | None = None, now: float | None = None) -> None:
        if self.output_token_ids[place] != self.UNREAD_TOKEN:
            raise ValueError(f"sequence {self.request_id!r}: output token {place} is already known")
        self.output_token_ids[place] = int(token_id)
        if logprob is not None:
            self.output_logprobs.append(float(logprob))
        if self.timing.t_first_token is None:
            self.timing.t_first_token = time.perf_counter() if now is None else now

    def drop_unread_token(self, place: int) -> None:
        """Forget a place whose token will not be read (the request was aborted meanwhile)."""
        if place < len(self.output_token_ids) and self.output_token_ids[place] == self.UNREAD_TOKEN:
            del self.output_token_ids[place:]

    def check_stop(self, token_id: int, *, eos_token_ids=frozenset()) -> FinishReason | None:
        """Whether the token just appended ends the request: a stop id, an end-of-sequence id
        unless ``ignore_eos``, or ``max_tokens`` reached (sequence.py:282-296).  The stop token
        stays in the output."""
        if token_id in self.sampling.stop_token_ids:
            return FinishReason.STOP
        if token_id in eos_token_ids and not self.sampling.ignore_eos:
            return FinishReason.STOP
        if self.num_output_tokens >= self.sampling.max_tokens:
            return FinishReason.LENGTH
        return None

    def finish(self, reason: FinishReason, *, now: float | None = None, stop_token_id: int | None = None) -> None:
        self.status = SeqStatus.FINISHED
        self.finish_reason = reason
        self.stop_token_id = stop_token_id
        self.timing.t_finished = time.perf_counter() if now is None else now
