"""The step function: a flat batch of (request, its next tokens) in, logits at the wanted
places out.

It runs only the tokens it is given, as one batch, against what earlier steps left in the
cache; it samples nothing and owns no request state.  Generation, replay and measurement all
go through it.  The reference's counterpart is ``ModelRunner.execute``
(src/turboserve/engine/runtime/worker.py:237-266), which also samples; its separable phases
(:180-233) are ``build_context`` / ``forward`` / ``logits`` here.
"""

from __future__ import annotations

from collections.abc import Sequence

import torch

from turboserve_amd.cache.layout import CacheLayout
from turboserve_amd.cache.storage import CacheStorage
from turboserve_amd.engine.batch import StepContext, StepEntry, StepLimits, build_context, validate_entries
from turboserve_amd.engine.decode_graph import DecodeGraphs
from turboserve_amd.models.decoder import DecoderModel


class ModelRunner:
    def __init__(self, model: DecoderModel, storage: CacheStorage, *, check: bool = True,
                 use_graphs: bool = True, max_graph_batch: int = 128) -> None:
        self.model = model
        self.storage = storage
        self.layout: CacheLayout = storage.layout
        self.check = check
        self.views = storage.views()
        self.vocab_size = model.plan.vocab_size
        self.num_steps = 0
        #: What a checked step's page ids, slots, token ids and state slots must lie inside.
        self.limits = StepLimits(
            num_pages=tuple(storage.num_pages), windows=tuple(self.layout.windows()),
            vocab_size=self.vocab_size, num_state_slots=storage.num_state_slots,
        )
        #: Steps of single tokens are replayed as HIP graphs (see ``decode_graph``), unless a part
        #: of the model says it cannot be recorded (``Part.capturable``).
        self.graphs: DecodeGraphs | None = None
        #: Fields the model's parts add to every step's packed buffer.
        self.extra_fields = model.step_fields()
        if use_graphs and model.is_capturable():
            self.graphs = DecodeGraphs(
                model, self.views, page_size=storage.page_size, num_groups=len(self.layout.groups),
                pad_state_slot=storage.pad_state_slot, max_batch=max_graph_batch, limits=self.limits,
                extra_fields=self.extra_fields,
            )

    def release(self) -> None:
        """Drop the cache tensors (the engine is closing)."""
        self.views = []
        self.storage = None
        if self.graphs is not None:
            self.graphs.release()
            self.graphs = None

    def context_for(self, entries: Sequence[StepEntry]) -> StepContext:
        """The packed step on the device.  With ``check`` (always, except in measurements)
        nothing a kernel would dereference leaves the host unchecked: token ids, page ids,
        slots and state slots are validated against the vocabulary and the pools first."""
        return build_context(
            entries,
            num_groups=len(self.layout.groups),
            page_size=self.storage.page_size,
            device=self.model.runtime.device,
            check=self.check,
            limits=self.limits,
            extra_fields=self.extra_fields,
        )

    @torch.inference_mode()
    def step(self, entries: Sequence[StepEntry], *, fresh_state_slots: Sequence[int] = (),
             tokens_from: tuple[torch.Tensor, dict[int, int]] | None = None) -> torch.Tensor:
        """Run one step and return 32-bit logits ``[wanted, V]`` on the device, in the order of
        the entries and of each entry's ``want``.  A step that wants nothing still runs (it
        fills the cache, worker.py:248-256) and returns ``[0, V]``.

        ``tokens_from = (source, {entry index: element})``: the single token of those entries
        is element ``element`` of the int32 device tensor ``source`` (what the step before
        sampled, not read back yet); only steps that replay as a graph take it
        (``takes_tokens_from``)."""
        self.storage.zero_state_slots(fresh_state_slots)
        device = self.model.runtime.device
        if not entries:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=device)
        if self.graphs is not None and self.graphs.accepts(entries):
            return self._graph_step(entries, tokens_from)
        if tokens_from is not None:
            raise ValueError("only a step of single tokens that replays as a graph can take tokens from the device")
        ctx = self.context_for(entries)
        stream = self.model.forward(ctx.token_ids, ctx, self.views)
        self.num_steps += 1
        if ctx.num_logit_rows == 0:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=device)
        return self.model.logits(stream, ctx.logit_rows)

    @torch.inference_mode()
    def dry_run(self, num_tokens: int) -> None:
        """One step of a made-up prompt of ``num_tokens`` tokens that writes nothing into the
        cache (every slot is the skip mark) and whose result is dropped: it makes every product
        of the model run once at that size, for warming up or for timing the library's kernels
        (the tokens differ from one another: products of equal rows draw less power and run
        faster than those of a real prompt, and would be timed at clocks serving never sees)."""
        page = self.storage.page_size
        groups = len(self.layout.groups)
        entry = StepEntry(
            request="dry-run", tokens=[(7919 * i + 13) % self.vocab_size for i in range(num_tokens)], start=0,
            tables=[[0] * (-(-num_tokens // page))] * groups, slots=[[-1] * num_tokens] * groups,
            state_slot=self.storage.pad_state_slot, want=[num_tokens - 1],
        )
        ctx = build_context([entry], num_groups=groups, page_size=page, device=self.model.runtime.device, check=False,
                            extra_fields=self.extra_fields)
        stream = self.model.forward(ctx.token_ids, ctx, self.views)
        self.model.logits(stream, ctx.logit_rows)
        torch.cuda.synchronize(self.model.runtime.device)

    def takes_tokens_from(self, num_entries: int) -> bool:
        """Whether a step of ``num_entries`` single tokens would replay as a graph."""
        return self.graphs is not None and 0 < num_entries <= self.graphs.max_batch

    def _graph_step(self, entries: Sequence[StepEntry], tokens_from=None) -> torch.Tensor:
        """A step of single tokens through its recorded graph.  The result is the graph's own
        buffer (or rows gathered from it): read it before the next step."""
        if self.check:
            validate_entries(entries, len(self.layout.groups), self.storage.page_size)
        logits = self.graphs.run(entries, tokens_from=tokens_from, check=self.check)
        self.num_steps += 1
        wanted = [i for i, entry in enumerate(entries) if len(entry.want) > 0]
        if len(wanted) == len(entries):
            return logits
        if not wanted:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=logits.device)
        return logits.index_select(0, torch.tensor(wanted, dtype=torch.long, device=logits.device))
