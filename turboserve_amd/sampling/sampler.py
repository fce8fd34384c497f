"""Batched sampling with per-request options (src/turboserve/engine/core/sampler.py:171-297).

The stages and their order are the reference's (penalty, log-probabilities, temperature,
top-k, top-p, draw); they run in one HIP kernel launch for the whole batch, one block per row.
A request's randomness is its own: the draw for its n-th token uses a counter-based generator
keyed by the request's seed with counter n, so a row does not depend on its batch neighbours
or on any global generator state (the property the reference gets from per-request
``torch.Generator`` objects, sampler.py:258-297), and a request that was preempted and
recomputed continues with the same numbers.
"""

from __future__ import annotations

from collections.abc import Sequence as SequenceABC
from dataclasses import dataclass

import numpy as np
import torch

from turboserve_amd.engine.sequence import Sequence
from turboserve_amd.sampling.params import SamplingParams


@dataclass
class SamplerOutput:
    token_ids: list[int]
    logprobs: list[float] | None = None  # nan for rows that did not ask (sampler.py:66-74)


class PendingSample:
    """What a sampling launch left on the device.  The copy to (pinned) host memory is queued
    right behind the sampler, with an event after it, so that ``read()`` waits for exactly this
    and not for whatever the stream was given afterwards (a step launched ahead)."""

    def __init__(self, tokens: torch.Tensor | None, logprobs: torch.Tensor | None,
                 params: SequenceABC[SamplingParams] = ()) -> None:
        self.tokens = tokens        # int32 [n] where it was computed, or None for no rows
        self.logprobs = logprobs    # float32 [n] or None
        self.params = params
        self._host_tokens = self._host_logprobs = self._event = None
        if tokens is not None and tokens.is_cuda:
            self._host_tokens = torch.empty(tokens.shape, dtype=tokens.dtype, pin_memory=True)
            self._host_tokens.copy_(tokens, non_blocking=True)
            if logprobs is not None:
                self._host_logprobs = torch.empty(logprobs.shape, dtype=logprobs.dtype, pin_memory=True)
                self._host_logprobs.copy_(logprobs, non_blocking=True)
            self._event = torch.cuda.Event()
            self._event.record(torch.cuda.current_stream(tokens.device))

    def read(self) -> SamplerOutput:
        if self.tokens is None:
            return SamplerOutput(token_ids=[])
        if self._event is not None:
            self._event.synchronize()
        tokens = self._host_tokens if self._host_tokens is not None else self.tokens
        out = SamplerOutput(token_ids=tokens.tolist())
        if self.logprobs is not None:
            values = (self._host_logprobs if self._host_logprobs is not None else self.logprobs).tolist()
            out.logprobs = [v if p.logprobs else float("nan") for v, p in zip(values, self.params)]
        return out


class Sampler:
    #: ``launch`` takes ``unread``: a row's history may end in a token only the device knows yet.
    takes_unread = True

    def __init__(self, ops) -> None:
        self.ops = ops

    def sample(
        self,
        logits: torch.Tensor,
        params: SequenceABC[SamplingParams],
        seeds: SequenceABC[int],
        draw_indices: SequenceABC[int],
        histories: SequenceABC[SequenceABC[int]] | None = None,
    ) -> SamplerOutput:
        """One token per row of ``logits [n, V]`` (32-bit, left untouched).

        ``seeds[i]`` / ``draw_indices[i]``: key and counter of row ``i``'s draw.
        ``histories[i]``: prompt + output tokens, read only when the row has a repetition
        penalty other than 1."""
        return self.launch(logits, params, seeds, draw_indices, histories).read()

    def launch(
        self,
        logits: torch.Tensor,
        params: SequenceABC[SamplingParams],
        seeds: SequenceABC[int],
        draw_indices: SequenceABC[int],
        histories: SequenceABC[SequenceABC[int]] | None = None,
        unread: tuple[torch.Tensor, SequenceABC[int]] | None = None,
    ) -> PendingSample:
        """``sample`` without the wait: the kernels are launched and the tokens stay on the
        device until ``PendingSample.read``.  ``unread``: the tokens of a launch whose result has
        not been read (int32 on the device) and, per row, the place in them of the row's own last
        token, or -1; a row with a repetition penalty counts that token into its history (where
        its ``histories`` entry has a negative stand-in)."""
        rows = int(logits.shape[0])
        if len(params) != rows or len(seeds) != rows or len(draw_indices) != rows:
            raise ValueError(f"{len(params)} params / {len(seeds)} seeds / {len(draw_indices)} counters for {rows} rows")
        if histories is not None and len(histories) != rows:
            raise ValueError(f"{len(histories)} histories for {rows} rows of logits")
        if unread is not None and len(unread[1]) != rows:
            raise ValueError(f"{len(unread[1])} places of unread tokens for {rows} rows of logits")
        if rows == 0:
            return PendingSample(None, None)
        if all(p.is_plain_greedy for p in params):
            return PendingSample(self.ops.argmax(logits), None, params)

        want_logprobs = any(p.logprobs for p in params)
        history_start = [0]
        pieces: list[np.ndarray] = []
        for i, p in enumerate(params):
            held = history_start[-1]
            if p.repetition_penalty != 1.0 and histories is not None:
                pieces.append(np.asarray(histories[i], dtype=np.int32))  # no copy where it is an int32 array already
                held += pieces[-1].shape[0]
            history_start.append(held)
        flat_history = np.concatenate(pieces) if pieces else np.empty(0, dtype=np.int32)
        floats = np.asarray(
            [[p.temperature for p in params], [p.top_p for p in params], [p.repetition_penalty for p in params]],
            dtype=np.float32,
        )
        seeds64 = np.asarray([int(s) & 0xFFFFFFFFFFFFFFFF for s in seeds], dtype=np.uint64)
        packed = np.concatenate([
            floats.reshape(-1).view(np.int32),
            np.asarray([p.top_k for p in params], dtype=np.int32),
            (seeds64 & np.uint64(0xFFFFFFFF)).astype(np.uint32).view(np.int32),
            (seeds64 >> np.uint64(32)).astype(np.uint32).view(np.int32),
            np.asarray([int(d) & 0xFFFFFFFF for d in draw_indices], dtype=np.uint32).view(np.int32),
            np.asarray(history_start, dtype=np.int32),
            np.asarray(unread[1] if unread is not None else [-1] * rows, dtype=np.int32),
            flat_history,
        ])
        # One copy, from pinned memory and queued on the stream: a copy from pageable memory
        # would make the host wait for everything the stream holds, a step launched ahead included.
        device = logits.device
        if device.type == "cuda":
            staged = torch.empty(packed.shape, dtype=torch.int32, pin_memory=True)
            staged.numpy()[:] = packed
            on_device = staged.to(device, non_blocking=True)
        else:
            on_device = torch.from_numpy(packed).to(device)
        temperature, top_p, penalty, top_k, seed_lo, seed_hi, draw, hstart, unread_row, hist = torch.split(
            on_device, [rows, rows, rows, rows, rows, rows, rows, rows + 1, rows, len(flat_history)]
        )
        tokens, logprobs = self.ops.sample(
            logits, temperature.view(torch.float32), top_k, top_p.view(torch.float32), penalty.view(torch.float32),
            seed_lo, seed_hi, draw, hist, hstart, want_logprobs,
            unread_tokens=unread[0] if unread is not None else None,
            unread_row=unread_row.contiguous() if unread is not None else None,
        )
        return PendingSample(tokens, logprobs, list(params))

    def sample_sequences(self, logits: torch.Tensor, sequences: SequenceABC[Sequence]) -> SamplerOutput:
        """Sample for requests: options, seed, draw counter (= tokens produced so far) and,
        only if a penalty is set, the token history of each (sampler.py:240-256)."""
        return self.launch_sequences(logits, sequences).read()

    def launch_sequences(self, logits: torch.Tensor, sequences: SequenceABC[Sequence],
                         unread: tuple[torch.Tensor, SequenceABC[int]] | None = None) -> PendingSample:
        """``sample_sequences`` without the wait.  ``unread``: see ``launch`` (a request whose last
        token is an unread one has ``Sequence.UNREAD_TOKEN`` there)."""
        return self.launch(
            logits,
            [seq.sampling for seq in sequences],
            [seq.sample_seed for seq in sequences],
            [seq.num_output_tokens for seq in sequences],
            [seq.token_array() if seq.sampling.repetition_penalty != 1.0 else () for seq in sequences],
            unread,
        )
