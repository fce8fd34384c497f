"""The engine loop: requests in, tokens out, one forward pass per ``step()``
(src/turboserve/engine/runtime/engine.py:118-508).

One process, one thread, one GPU.  ``step()`` = schedule, run the step function, sample, feed
the tokens back.  Every collaborator can be passed in, so a test can build an engine around a
tiny pool or a stand-in runner.
"""

from __future__ import annotations

import dataclasses
import logging
import time
from collections.abc import Sequence as SequenceABC
from dataclasses import dataclass, field
from typing import Any

import torch

from turboserve_amd.cache.manager import CacheManager
from turboserve_amd.cache.sizing import CacheSizing, activation_headroom_bytes, size_cache
from turboserve_amd.config.engine_config import EngineConfig
from turboserve_amd.engine.detokenizer import TextStream, get_tokenizer
from turboserve_amd.engine.outputs import RequestOutput
from turboserve_amd.engine.scheduler import Scheduler, SchedulerOutput
from turboserve_amd.engine.sequence import Sequence
from turboserve_amd.sampling.params import FinishReason, SamplingParams

logger = logging.getLogger(__name__)


@dataclass(frozen=True)
class EngineStats:
    """A snapshot of engine health (engine.py:80-115).  The two prefix-cache fields are in the
    reference's record and always zero here: there is no prefix cache."""

    num_running: int
    num_waiting: int
    num_preempted: int
    num_unfinished: int
    num_finished: int
    num_preemptions: int
    num_steps: int
    kv_utilization: float  # fraction of cache pages held by requests, the fullest group's
    prefix_hit_rate: float
    num_prompt_tokens: int
    num_generated_tokens: int
    num_cached_prompt_tokens: int

    def to_dict(self) -> dict[str, int | float]:
        return dataclasses.asdict(self)


@dataclass
class _InFlight:
    """A step that has been launched and whose sampled tokens are still on the device."""

    sampled: list  # the step's ScheduledSeq items that sample, in the order of the sampler's rows
    pending: Any   # sampler.PendingSample (or a stand-in with read()); None if nothing samples
    places: dict = field(default_factory=dict)  # seq_id -> place of this step's token in the request's output, if taken ahead


@dataclass
class _Sampled:
    """A sampler result that is already on the host, in the shape of a pending one."""

    result: Any

    def read(self):
        return self.result


class LLMEngine:
    def __init__(
        self,
        config: EngineConfig,
        *,
        model: Any | None = None,
        model_config: Any | None = None,
        tokenizer: Any | None = None,
        storage: Any | None = None,
        scheduler: Scheduler | None = None,
        runner: Any | None = None,
        sampler: Any | None = None,
        local_files_only: bool = True,
    ) -> None:
        # local_files_only: in the reference's signature (runtime/engine.py:125-146); this engine
        # reads local folders only, whatever its value.
        del local_files_only
        from turboserve_amd.cache.layout import CacheLayout
        from turboserve_amd.cache.storage import CacheStorage
        from turboserve_amd.engine.loading import load_model
        from turboserve_amd.engine.runner import ModelRunner
        from turboserve_amd.sampling.sampler import Sampler

        self.config = config
        if model is None:
            model_config, model, report = load_model(
                config.model, dtype=config.resolved_dtype(), device=config.resolved_device()
            )
            logger.info("weights: %s", report.summary())
        self.model = model
        self.model_config = model_config
        self.tokenizer = tokenizer if tokenizer is not None else get_tokenizer(config.tokenizer or config.model)
        self._eos_token_ids = self._resolve_eos_token_ids()

        self.sizing: CacheSizing | None = None
        sched_cfg = config.scheduler
        if storage is None and runner is None:
            layout = CacheLayout.from_model(model)
            runtime = model.runtime
            itemsize = torch.empty((), dtype=runtime.dtype).element_size()
            activation = 0
            if sched_cfg.num_blocks is None:
                activation = activation_headroom_bytes(model, sched_cfg, itemsize)
            self.sizing = size_cache(
                layout, sched_cfg, itemsize=itemsize, activation_bytes=activation,
                gpu_memory_utilization=config.gpu_memory_utilization, max_model_len=config.max_model_len,
                device=runtime.device,
            )
            storage = CacheStorage(layout, self.sizing.num_blocks, sched_cfg.block_size, sched_cfg.max_num_seqs,
                                   runtime.dtype, runtime.device)
        self.storage = storage
        if scheduler is None:
            if storage is None:
                raise ValueError("an engine built around a stand-in runner needs its scheduler passed in")
            cache = CacheManager(storage.layout.windows(), storage.num_pages, sched_cfg.block_size, sched_cfg.max_num_seqs)
            scheduler = Scheduler(sched_cfg, cache)
        self.scheduler = scheduler
        self.runner = runner if runner is not None else ModelRunner(model, storage)
        self.sampler = sampler if sampler is not None else Sampler(model.runtime.ops)
        if (config.tune_gemm_tokens or config.tune_gemm_step_sizes) and runner is None:
            self._tune_library_products()
        self._decoders: dict[str, TextStream] = {}
        self._seed = config.seed if config.seed is not None else time.time_ns() & 0xFFFFFFFF
        self._num_generated_tokens = 0
        self._num_prompt_tokens = 0
        self._closed = False
        self._in_flight: _InFlight | None = None  # a step launched ahead whose tokens have not been read

    # -- helpers --------------------------------------------------------------------------------

    @classmethod
    def from_env(cls, environ=None, **kwargs: Any) -> "LLMEngine":
        """An engine built from the ``TURBOSERVE_*`` variables (engine.py:218-221 builds one
        from the reference's settings object, which reads the same variables)."""
        return cls(EngineConfig.from_env(environ), **kwargs)

    def _tune_library_products(self) -> None:
        """Time the BLAS library's kernels for this model's projections at the configured step
        sizes (dry steps that leave the cache alone) and keep the fastest."""
        if self.model.runtime.dtype != torch.bfloat16:
            return  # the 32-bit path uses this engine's own product kernel
        from turboserve_amd.kernels.gemm_tuning import LibraryGemmTuning, OwnProductChoices

        budget = self.config.scheduler.max_num_batched_tokens
        sizes = {min(t, budget) for t in self.config.tune_gemm_tokens}
        if self.config.tune_gemm_step_sizes:
            ops = self.model.runtime.ops
            ops.library_buckets = ops.bucket_sizes(budget)  # until close(): the model may outlive this engine
            sizes.update(size for size in ops.library_buckets if size > ops.skinny_max_rows)
        started = time.perf_counter()
        ops = self.model.runtime.ops
        own_rows = ops.wide_default_rows
        try:
            # First the library's kernels for every product (this engine's own product for steps of
            # many rows stands aside meanwhile) ...
            ops.wide_default_rows = 0
            with LibraryGemmTuning(self.config.gemm_tuning_file) as tuning:
                for tokens in sorted(sizes):
                    self.runner.dry_run(tokens)
            # ... then, with the library's winners in use and its timing mode off, every such
            # product runs both ways, by the library and by this engine's own kernel, and the
            # faster one is kept (``Ops.wide_choices``; what an earlier process found is read
            # from a file beside the library's results and not timed again).
            choices = OwnProductChoices(tuning.results_file, ops)
            choices.load()
            ops.time_wide_choices = True
            for tokens in sorted(sizes):
                self.runner.dry_run(tokens)
            choices.save()
        finally:
            ops.time_wide_choices = False
            ops.wide_default_rows = own_rows
        logger.info("library products timed for steps of %s tokens in %.1f s (%d choices kept in %s)",
                    sorted(sizes), time.perf_counter() - started, tuning.num_results(), tuning.results_file)

    def _resolve_eos_token_ids(self) -> frozenset[int]:
        """Every id that ends a generation: the checkpoint configuration's and the tokenizer's
        (engine.py:223-237; the two differ for chat checkpoints, whose tokenizer ends a turn
        with a token that ``config.json`` does not list)."""
        ids = {int(i) for i in (getattr(self.model_config, "eos_token_ids", ()) or ())}
        named = getattr(self.tokenizer, "eos_token_id", None)
        if isinstance(named, int) and not isinstance(named, bool):
            ids.add(named)
        elif isinstance(named, (list, tuple)):
            ids.update(int(i) for i in named)
        return frozenset(ids)

    @property
    def eos_token_ids(self) -> frozenset[int]:
        return self._eos_token_ids

    def encode(self, prompt: str) -> list[int]:
        if self.tokenizer is None:
            raise TypeError("no tokenizer is configured: pass prompts as token ids")
        return [int(t) for t in self.tokenizer.encode(prompt, add_special_tokens=False)]

    def _request_seed(self, sampling: SamplingParams, seq_index: int) -> int:
        """A request's own seed, or one derived from the engine's seed and its arrival number."""
        if sampling.seed is not None:
            return int(sampling.seed) & 0xFFFFFFFFFFFFFFFF
        return ((self._seed & 0xFFFFFFFF) << 32 | (seq_index & 0xFFFFFFFF)) ^ 0x9E3779B97F4A7C15

    # -- requests -------------------------------------------------------------------------------

    def add_request(
        self,
        request_id: str,
        prompt: str | SequenceABC[int],
        sampling: SamplingParams | None = None,
        *,
        priority: int = 0,
        arrival: float | None = None,
    ) -> Sequence:
        """Queue a request given as text or as token ids (engine.py:283-323)."""
        if self._closed:
            raise RuntimeError("engine is closed")
        token_ids = self.encode(prompt) if isinstance(prompt, str) else [int(t) for t in prompt]
        if not token_ids:
            raise ValueError(f"request {request_id!r} has an empty prompt")
        plan = getattr(self.model, "plan", None)
        vocab = None if plan is None else plan.vocab_size
        if vocab is not None and any(not 0 <= t < vocab for t in token_ids):
            raise ValueError(f"request {request_id!r} has a token id outside the vocabulary of {vocab}")
        sampling = sampling or SamplingParams()
        seq = self.scheduler.add_request(
            request_id, token_ids, sampling, priority=priority, arrival=arrival,
            sample_seed=self._request_seed(sampling, self.scheduler._next_seq_id),
        )
        self._decoders[request_id] = TextStream(self.tokenizer, sampling.stop)
        self._num_prompt_tokens += len(token_ids)
        return seq

    def abort(self, request_id: str, *, now: float | None = None) -> bool:
        self._decoders.pop(request_id, None)
        return self.scheduler.abort(request_id, now=now)

    def has_unfinished(self) -> bool:
        return self.scheduler.has_unfinished()

    # -- the step -------------------------------------------------------------------------------

    def step(self, *, now: float | None = None) -> list[RequestOutput]:
        """Advance every scheduled request.  An empty list is normal: nothing queued, only
        unfinished portions of prompts ran, or everything scheduled was preempted
        (engine.py:340-356).

        With ``config.run_ahead`` a decode step is launched before the tokens of the step before
        it have been read (``_run_ahead``); a call then returns the outputs of the step that was
        launched by the call before it."""
        if self._closed:
            raise RuntimeError("engine is closed")
        timestamp = time.perf_counter() if now is None else now
        outputs: list[RequestOutput] = []
        flight, self._in_flight = self._in_flight, None
        if flight is None:
            scheduled = self.scheduler.schedule(now=timestamp)
            outputs.extend(self._output_for_dropped(seq) for seq in scheduled.dropped)
            if scheduled.is_empty:
                return outputs
            flight = self._launch(scheduled)
        if self.config.run_ahead:
            self._in_flight = self._run_ahead(flight, outputs, now=timestamp)
        outputs.extend(self._collect(flight, now=now))
        return outputs

    def _launch(self, scheduled: SchedulerOutput, tokens_from=None) -> "_InFlight":
        """Start a step on the GPU: the model, then the sampler; nothing is waited for."""
        entries = scheduled.entries()
        if tokens_from is None:
            logits = self.runner.step(entries, fresh_state_slots=scheduled.fresh_state_slots)
        else:  # only a runner that said it takes them (`takes_tokens_from`) is asked to
            logits = self.runner.step(entries, fresh_state_slots=scheduled.fresh_state_slots, tokens_from=tokens_from)
        sampled = scheduled.sampled()
        unread = None
        if tokens_from is not None and sampled and getattr(self.sampler, "takes_unread", False):
            # Every request of a step launched ahead has its last token still on the device; a
            # repetition penalty must see it.
            tokens, patch = tokens_from
            row_of = {id(item): index for index, item in enumerate(scheduled.scheduled)}
            unread = (tokens, [patch.get(row_of[id(item)], -1) for item in sampled])
        pending = self._launch_sampler(logits, [item.seq for item in sampled], unread) if sampled else None
        return _InFlight(sampled, pending)

    def _launch_sampler(self, logits, sequences, unread=None):
        launch = getattr(self.sampler, "launch_sequences", None)
        if launch is not None:
            return launch(logits, sequences, unread) if unread is not None else launch(logits, sequences)
        return _Sampled(self.sampler.sample_sequences(logits, sequences))  # a stand-in sampler without a launch/read split

    def _run_ahead(self, flight: "_InFlight", outputs: list[RequestOutput], *, now: float) -> "_InFlight | None":
        """Schedule and launch the step after ``flight`` while ``flight`` still runs.

        Possible when that step is known without the tokens' values: the unfinished requests of
        ``flight`` all sample and are all the running requests, nothing waits to be admitted,
        and the step replays as a graph (a repetition penalty gets the unread token on the device).  Each request
        gets a place for its unread token (unless that token is its last by ``max_tokens``: then
        it has no part in the next step); the step's token ids are copied on the device from the
        sampler's result.  A request that then turns out to have ended (a stop token, a stop
        string, an abort) leaves a row in the launched step whose result is dropped."""
        source = {item.seq.seq_id: row for row, item in enumerate(flight.sampled) if not item.seq.is_finished}
        live = [item.seq for item in flight.sampled if not item.seq.is_finished]
        tokens = getattr(flight.pending, "tokens", None)
        if not live or tokens is None:
            return None
        takes = getattr(self.runner, "takes_tokens_from", None)
        if takes is None or not takes(len(live)) or not self.scheduler.only_running(live):
            return None
        if any(seq.sampling.repetition_penalty != 1.0 for seq in live) and not getattr(self.sampler, "takes_unread", False):
            return None  # the penalty needs the unread token, and this sampler cannot be given it
        for seq in live:
            # A request that reaches max_tokens with the token in flight takes no place: it has
            # nothing to compute in the next step and ends when its token is read.
            if seq.num_output_tokens + 1 < seq.sampling.max_tokens:
                flight.places[seq.seq_id] = seq.append_unread_token()
        scheduled = self.scheduler.schedule(now=now)
        outputs.extend(self._output_for_dropped(seq) for seq in scheduled.dropped)
        if scheduled.is_empty:
            return None
        patch = {}
        for index, item in enumerate(scheduled.scheduled):
            if item.num_new_tokens != 1 or item.seq.seq_id not in source:
                raise RuntimeError("the step scheduled ahead holds something other than the running requests' next tokens")
            patch[index] = source[item.seq.seq_id]
        return self._launch(scheduled, tokens_from=(tokens, patch))

    def _collect(self, flight: "_InFlight", *, now: float | None) -> list[RequestOutput]:
        """Wait for a launched step's tokens and feed them back: stop checks, text, per-request
        deltas (engine.py:366-410)."""
        if flight.pending is None:
            return []
        result = flight.pending.read()
        if now is None:  # the tokens exist from here on, not from when the call began
            now = time.perf_counter()
        tokens, logprobs = result.token_ids, result.logprobs
        outputs = []
        for index, (item, token) in enumerate(zip(flight.sampled, tokens)):
            seq = item.seq
            if seq.is_finished:
                # aborted meanwhile, or ended by the step before this one was launched ahead of
                if seq.seq_id in flight.places:
                    seq.drop_unread_token(flight.places[seq.seq_id])
                continue
            logprob = None
            if logprobs is not None and seq.sampling.logprobs:
                logprob = logprobs[index]
            place = flight.places.get(seq.seq_id)
            if place is None:
                reason = self.scheduler.append_token(seq, token, eos_token_ids=self._eos_token_ids, logprob=logprob, now=now)
            else:
                reason = self.scheduler.resolve_token(seq, place, token, eos_token_ids=self._eos_token_ids,
                                                      logprob=logprob, now=now)
            outputs.append(self._emit(seq, token, reason, logprob, now=now))
        self._num_generated_tokens += len(outputs)
        return outputs

    def _emit(self, seq: Sequence, token: int, reason, logprob, *, now: float) -> RequestOutput:
        decoder = self._decoders.get(seq.request_id)
        if decoder is None:
            decoder = self._decoders[seq.request_id] = TextStream(self.tokenizer, seq.sampling.stop)
        delta = decoder.push((token,))
        text = delta.text
        if delta.stopped and reason is None:
            self.scheduler.finish(seq, FinishReason.STOP, now=now)
            reason = FinishReason.STOP
        elif reason is not None and not delta.stopped:
            text += decoder.close()
        if reason is not None:
            self._decoders.pop(seq.request_id, None)
        return RequestOutput(
            request_id=seq.request_id, new_token_ids=[token], text_delta=text, finished=reason is not None,
            finish_reason=reason, timing=seq.timing, prompt_tokens=seq.num_prompt_tokens,
            output_tokens=seq.num_output_tokens, logprobs=[] if logprob is None else [logprob],
        )

    def _output_for_dropped(self, seq: Sequence) -> RequestOutput:
        self._decoders.pop(seq.request_id, None)
        return RequestOutput(
            request_id=seq.request_id, finished=True, finish_reason=seq.finish_reason, timing=seq.timing,
            prompt_tokens=seq.num_prompt_tokens, output_tokens=seq.num_output_tokens,
        )

    # -- convenience ----------------------------------------------------------------------------

    def generate(
        self,
        prompts: SequenceABC[str | SequenceABC[int]],
        sampling: SamplingParams | SequenceABC[SamplingParams] | None = None,
        *,
        request_id_prefix: str = "gen",
    ) -> list[RequestOutput]:
        """Run prompts to completion; one aggregate result each, in input order (engine.py:414-448)."""
        order = []
        for index, prompt in enumerate(prompts):
            request_id = f"{request_id_prefix}-{index}"
            params = sampling[index] if isinstance(sampling, (list, tuple)) else sampling
            self.add_request(request_id, prompt, params)
            order.append(request_id)
        merged: dict[str, RequestOutput] = {}
        while self.has_unfinished():
            for output in self.step():
                current = merged.get(output.request_id)
                if current is None:
                    merged[output.request_id] = output
                    continue
                current.new_token_ids.extend(output.new_token_ids)
                current.logprobs.extend(output.logprobs)
                current.text_delta += output.text_delta
                current.finished = output.finished
                current.finish_reason = output.finish_reason
                current.output_tokens = output.output_tokens
                current.timing = output.timing
        return [merged[request_id] for request_id in order if request_id in merged]

    # -- observability --------------------------------------------------------------------------

    @property
    def device(self) -> torch.device:
        return self.model.runtime.device

    @property
    def dtype(self) -> torch.dtype:
        return self.model.runtime.dtype

    def engine_stats(self) -> EngineStats:
        """Structured snapshot (engine.py:452-468)."""
        raw = self.scheduler.stats()
        utilization = 0.0
        for pool in self.scheduler.cache.pools:
            if pool.num_pages:
                utilization = max(utilization, pool.num_in_use / pool.num_pages)
        return EngineStats(
            num_running=int(raw["num_running"]), num_waiting=int(raw["num_waiting"]),
            num_preempted=int(raw["num_preempted"]), num_unfinished=int(raw["num_unfinished"]),
            num_finished=int(raw["num_finished"]), num_preemptions=int(raw["num_preemptions"]),
            num_steps=int(raw["num_steps"]), kv_utilization=utilization, prefix_hit_rate=0.0,
            num_prompt_tokens=self._num_prompt_tokens, num_generated_tokens=self._num_generated_tokens,
            num_cached_prompt_tokens=0,
        )

    def stats(self) -> dict[str, int | float | str]:
        """Flat, JSON-safe counters (engine.py:470-484)."""
        out: dict[str, int | float | str] = dict(self.scheduler.stats())
        out.update(self.engine_stats().to_dict())
        out["model"] = self.config.model
        runtime = getattr(self.model, "runtime", None)
        if runtime is not None:
            out["device"] = str(runtime.device)
            out["dtype"] = str(runtime.dtype).removeprefix("torch.")
        if self.storage is not None:
            out["block_size"] = self.storage.page_size
            out["num_kv_blocks"] = min(self.storage.num_pages) if self.storage.num_pages else 0
            out["kv_bytes"] = self.storage.num_bytes()
        return out

    def close(self) -> None:
        if self._closed:
            return
        self._closed = True
        self._in_flight = None
        self.scheduler.reset()
        self._decoders.clear()
        self.storage = None
        if self.runner is not None and hasattr(self.runner, "release"):
            self.runner.release()
        if self.config.tune_gemm_step_sizes and self.model is not None:
            self.model.runtime.ops.library_buckets = ()
        if torch.cuda.is_available():
            torch.cuda.empty_cache()

    def __enter__(self) -> "LLMEngine":
        return self

    def __exit__(self, *exc: object) -> None:
        self.close()
