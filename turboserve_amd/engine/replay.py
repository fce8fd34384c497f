"""Trace replay: feed given token ids through the model step by step and write logits.

It samples nothing and has no forward pass, cache or loader of its own: it drives the same
model, step function, cache manager and kernels that generation uses.  The reference has no
such program; its nearest parts are the test helpers that call the model with hand-built
metadata (tests/unit/test_model_parity.py:40-133).

Input, one JSON object a line::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step that wants something, ``<out>/<step>.f32`` holds the logits at the wanted places,
little-endian 32-bit floats ``[wanted, vocab]``, in the order of the entries and of ``want``.
After every step a line ``done <step>`` is printed and flushed.
"""

from __future__ import annotations

import json
import sys
from collections.abc import Iterable
from pathlib import Path
from typing import IO, Any

from turboserve_amd.cache.manager import CacheManager
from turboserve_amd.engine.batch import StepEntry
from turboserve_amd.engine.loading import build_storage, load_model
from turboserve_amd.engine.runner import ModelRunner

#: ``max_tokens`` counts every live request's tokens rounded up to this (or to the page size, if
#: that is larger).
TOKEN_ROUNDING = 64
#: Requests that may be live at once unless the caller says otherwise.
DEFAULT_MAX_LIVE = 4


class TraceReplayer:
    def __init__(self, model_dir: str | Path, *, dtype: str, max_tokens: int, page_size: int = 16,
                 max_live: int = DEFAULT_MAX_LIVE, device: str = "cuda:0") -> None:
        if page_size < 1 or page_size & (page_size - 1):
            raise ValueError(f"page_size must be a power of two, got {page_size}")
        if max_tokens < 1:
            raise ValueError("--max-tokens must be positive")
        if max_live < 1:
            raise ValueError("--max-live must be positive")
        self.config, self.model, self.report = load_model(model_dir, dtype=dtype, device=device)
        rounding = max(TOKEN_ROUNDING, page_size)
        num_pages = -(-max_tokens // rounding) * (rounding // page_size)
        self.max_live = max_live
        self.storage = build_storage(self.model, num_pages, page_size, max_live)
        self.manager = CacheManager(self.storage.layout.windows(), num_pages, page_size, max_live)
        self.runner = ModelRunner(self.model, self.storage)

    def run_step(self, record: dict[str, Any]):
        """Run one step record; returns the device logits ``[wanted, V]`` (possibly empty)."""
        entries: list[StepEntry] = []
        fresh: list[int] = []
        for item in record.get("entries", []):
            request = item["id"]
            tokens = [int(t) for t in item["tokens"]]
            if not self.manager.has(request):
                fresh.append(self.manager.admit(request).state_slot)
            held = self.manager.get(request)
            start = held.num_tokens
            slots = self.manager.append(request, len(tokens))
            entries.append(StepEntry(
                request=request, tokens=tokens, start=start, tables=held.tables, slots=slots,
                state_slot=held.state_slot, want=[int(w) for w in item.get("want", [])],
            ))
        logits = self.runner.step(entries, fresh_state_slots=fresh)
        for request in record.get("end", []):
            if self.manager.has(request):
                self.manager.free(request)
        return logits

    def replay(self, lines: Iterable[str], out_dir: str | Path, done: IO[str] = sys.stdout) -> None:
        out = Path(out_dir)
        out.mkdir(parents=True, exist_ok=True)
        for line in lines:
            line = line.strip()
            if not line:
                continue
            record = json.loads(line)
            step = record["step"]
            logits = self.run_step(record)
            if logits.shape[0] > 0:
                logits.detach().to("cpu").contiguous().numpy().astype("<f4", copy=False).tofile(out / f"{step}.f32")
            print(f"done {step}", file=done, flush=True)


def main(argv: list[str] | None = None) -> int:
    import argparse

    parser = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    parser.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    parser.add_argument("--out", required=True, help="folder the <step>.f32 files are written to")
    parser.add_argument("--max-tokens", type=int, required=True,
                        help="most tokens live requests hold at once (each rounded up to 64); sizes the page pool")
    parser.add_argument("--page-size", type=int, default=16,
                        help="tokens per cache page, a power of two; above 64, --max-tokens counts in pages")
    parser.add_argument("--max-live", type=int, default=DEFAULT_MAX_LIVE, help="most requests live at once")
    args = parser.parse_args(argv)
    replayer = TraceReplayer(args.model, dtype=args.dtype, max_tokens=args.max_tokens, page_size=args.page_size,
                             max_live=args.max_live)
    replayer.replay(sys.stdin, args.out)
    return 0
