"""Decode steps as HIP graphs.

A step that brings one token for each of its requests launches a few hundred small kernels;
at a batch of one the launches, not the GPU, set the pace.  Such a step is therefore recorded
once per shape as a HIP graph (``torch.cuda.CUDAGraph``) over static buffers and replayed:
per step the host fills one pinned int32 buffer (the packed step of ``engine.batch``, in the
shape's layout), copies it to the device and launches the graph.

Shapes are bucketed so that few graphs serve every batch: the number of requests is rounded up
to a power of two (the extra rows are padding: position 0, context 1, no cache write, results
dropped) and each cache group's block-table width to a power of two.  The kernels read the
true context lengths from the device, so one graph serves every length up to its width.  What
the engine's own parts launch in such a step are this engine's kernels only (no BLAS call, no
memset node): products of up to 128 rows are the weight-streaming kernels, or, where K is no
multiple of 8, the plain fused-multiply-add kernel.  A part from elsewhere may record torch
operations; it answers for them with ``Part.capturable``.

The reference has no counterpart: it launches eager torch ops every step
(src/turboserve/engine/runtime/worker.py:221-233).
"""

from __future__ import annotations

from collections.abc import Sequence

import torch

from turboserve_amd.engine.batch import StepContext, StepEntry, StepLayout, StepLimits, check_packed, context_views, pack_step


def next_power_of_two(n: int) -> int:
    return 1 if n <= 1 else 1 << (n - 1).bit_length()


class _Graph:
    """One recorded shape: its static input buffer, context, output and the graph."""

    def __init__(self, batch: int, widths: tuple[int, ...], extra_fields=()) -> None:
        self.batch = batch
        self.widths = widths
        self.layout = StepLayout.make(batch, batch, batch, widths, extra_fields)
        self.graph: torch.cuda.CUDAGraph | None = None
        self.device_ints: torch.Tensor | None = None
        self.host_ints: list[torch.Tensor] = []
        self.turn = 0
        self.ctx: StepContext | None = None
        self.logits: torch.Tensor | None = None


class DecodeGraphs:
    def __init__(self, model, views, *, page_size: int, num_groups: int, pad_state_slot: int,
                 max_batch: int = 128, limits: StepLimits | None = None, extra_fields=()) -> None:
        self.model = model
        self.views = views
        self.page_size = page_size
        self.num_groups = num_groups
        self.pad_state_slot = pad_state_slot
        self.max_batch = max_batch
        #: What every replayed step's page ids, slots and token ids are checked against.
        self.limits = limits
        #: Fields the model's parts add to the packed buffer (``Part.step_fields``).
        self.extra_fields = tuple(extra_fields)
        self.device = model.runtime.device
        self._graphs: dict[tuple, _Graph] = {}
        self._pool = None
        self.num_replays = 0

    # -- shape -----------------------------------------------------------------------------------

    def accepts(self, entries: Sequence[StepEntry]) -> bool:
        return 0 < len(entries) <= self.max_batch and all(len(e.tokens) == 1 for e in entries)

    def _key(self, entries: Sequence[StepEntry]) -> tuple:
        batch = next_power_of_two(len(entries))
        widths = tuple(
            max(4, next_power_of_two(max(len(e.tables[g]) for e in entries))) for g in range(self.num_groups)
        )
        return batch, widths

    # -- buffers ---------------------------------------------------------------------------------

    def _build(self, key: tuple) -> _Graph:
        batch, widths = key
        shape = _Graph(batch, widths, self.extra_fields)
        total = shape.layout.total
        shape.device_ints = torch.zeros(total, dtype=torch.int32, device=self.device)
        shape.host_ints = [torch.zeros(total, dtype=torch.int32).pin_memory() for _ in range(2)]
        max_context = max(widths) * self.page_size
        shape.ctx = StepContext(
            num_tokens=batch,
            num_seqs=batch,
            **context_views(shape.layout, shape.device_ints),
            query_lens=[1] * batch,
            context_lens_host=[max_context] * batch,
            max_query_len=1,
            max_context_len=max_context,
            num_logit_rows=batch,
            num_prefill_seqs=0,
            num_decode_seqs=batch,
            num_prefill_tokens=0,
            max_prefill_context_len=0,
            max_decode_context_len=max_context,
            recorded=True,
        )
        # Harmless contents for the eager warm-up and the recording: every row is padding.
        shape.device_ints.copy_(self._fill(shape, []))

        def run() -> torch.Tensor:
            stream = self.model.forward(shape.ctx.token_ids, shape.ctx, self.views)
            return self.model.logits(stream, shape.ctx.logit_rows)

        # Once eagerly on a side stream (tables grow, libraries load, allocator warms up), then record.
        side = torch.cuda.Stream(device=self.device)
        side.wait_stream(torch.cuda.current_stream(self.device))
        with torch.cuda.stream(side):
            run()
        torch.cuda.current_stream(self.device).wait_stream(side)
        torch.cuda.synchronize(self.device)
        shape.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(shape.graph, pool=self._pool):
            shape.logits = run()
        if self._pool is None:
            self._pool = shape.graph.pool()
        return shape

    def _fill(self, shape: _Graph, entries: Sequence[StepEntry], patch: dict[int, int] | None = None,
              check: bool = False) -> torch.Tensor:
        """Write a step into the next pinned buffer (the packer of every step, ``pack_step``);
        rows beyond the entries are padding.  ``patch[i] = j``: entry ``i`` takes its token from
        element ``j`` of a device tensor."""
        shape.turn ^= 1
        host = shape.host_ints[shape.turn]
        data = host.numpy()
        pack_step(data, shape.layout, entries, range(shape.batch), pad_state_slot=self.pad_state_slot, token_sources=patch,
                  recorded=True)
        if check and self.limits is not None:
            check_packed(data, shape.layout, entries, self.page_size, self.limits)
        return host

    # -- the step --------------------------------------------------------------------------------

    def run(self, entries: Sequence[StepEntry], *, tokens_from: tuple[torch.Tensor, dict[int, int]] | None = None,
            check: bool = True) -> torch.Tensor:
        """Replay the graph of the entries' shape; returns the graph's own 32-bit logits buffer
        ``[len(entries), V]`` (overwritten by the next replay of that shape).  ``tokens_from =
        (source, {entry index: element of source})``: those entries' token ids are not known on
        the host yet and are copied on the device from ``source`` (int32) before the replay.
        With ``check`` the packed step is validated before it is copied to the device."""
        key = self._key(entries)
        shape = self._graphs.get(key)
        if shape is None:
            shape = self._graphs[key] = self._build(key)
        host = self._fill(shape, entries, tokens_from[1] if tokens_from else None, check=check)
        shape.device_ints.copy_(host, non_blocking=True)
        if tokens_from and tokens_from[1]:
            self.model.runtime.ops.patch_tokens(shape.ctx.token_ids, shape.ctx.token_source, tokens_from[0])
        shape.graph.replay()
        self.num_replays += 1
        return shape.logits[: len(entries)]

    def release(self) -> None:
        self._graphs.clear()
        self._pool = None
