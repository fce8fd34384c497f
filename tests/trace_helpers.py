"""Builders of replay traces: the ways a set of requests can be cut into steps."""

from __future__ import annotations

from collections.abc import Sequence


def whole(requests: dict[str, list[int]]) -> list[dict]:
    """Each request alone and whole: one step each, every position wanted."""
    steps = []
    for step, (rid, tokens) in enumerate(requests.items()):
        steps.append({"step": step, "entries": [{"id": rid, "tokens": tokens, "want": list(range(len(tokens)))}],
                      "end": [rid]})
    return steps


def prefix_then_single(requests: dict[str, list[int]], tail: int = 32) -> list[dict]:
    """Most of each request in one step, then its last ``tail`` tokens one by one."""
    steps: list[dict] = []
    for rid, tokens in requests.items():
        head = max(1, len(tokens) - tail)
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": tokens[:head], "want": list(range(head))}],
                      "end": []})
        for pos in range(head, len(tokens)):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [tokens[pos]], "want": [0]}],
                          "end": [rid] if pos == len(tokens) - 1 else []})
        if head == len(tokens):
            steps[-1]["end"] = [rid]
    return steps


def portions(requests: dict[str, list[int]], sizes: Sequence[int]) -> list[dict]:
    """Each request alone, in portions whose sizes cycle through ``sizes`` (down to two tokens)."""
    steps: list[dict] = []
    for rid, tokens in requests.items():
        pos, k = 0, 0
        while pos < len(tokens):
            n = min(sizes[k % len(sizes)], len(tokens) - pos)
            k += 1
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": tokens[pos:pos + n],
                                                            "want": list(range(n))}],
                          "end": [rid] if pos + n == len(tokens) else []})
            pos += n
    return steps


def mixed(requests: dict[str, list[int]], sizes: Sequence[int], max_live: int = 4, decode_tail: int = 6,
          skip_every: int = 5) -> list[dict]:
    """Up to ``max_live`` requests at a time: each is fed in portions from ``sizes`` and its
    last ``decode_tail`` tokens one by one, so portions of some run beside single tokens of
    others; every ``skip_every``-th turn a live request sits a step out.  A request that ends
    frees its pages for the next one waiting."""
    waiting = list(requests.items())
    live: list[dict] = []
    steps: list[dict] = []
    turn = 0
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, tokens = waiting.pop(0)
            live.append({"id": rid, "tokens": tokens, "pos": 0, "k": len(live)})
        entries, ended = [], []
        for state in live:
            turn += 1
            if skip_every and turn % skip_every == 0 and len(live) > 1:
                continue  # left out of this step, goes on later
            remaining = len(state["tokens"]) - state["pos"]
            if remaining <= decode_tail:
                n = 1
            else:
                n = min(sizes[state["k"] % len(sizes)], remaining - decode_tail)
                state["k"] += 1
            chunk = state["tokens"][state["pos"]:state["pos"] + n]
            entries.append({"id": state["id"], "tokens": chunk, "want": list(range(n))})
            state["pos"] += n
            if state["pos"] == len(state["tokens"]):
                ended.append(state["id"])
        if not entries:
            continue
        steps.append({"step": len(steps), "entries": entries, "end": ended})
        live = [s for s in live if s["id"] not in ended]
    return steps


def collect(steps: list[dict], outputs: dict[int, "object"], requests: dict[str, list[int]]):
    """Reassemble per-request ``[len, V]`` logits from per-step outputs (``outputs[step]`` is a
    ``[wanted, V]`` tensor)."""
    import torch

    rows: dict[str, list] = {rid: [None] * len(tokens) for rid, tokens in requests.items()}
    pos = {rid: 0 for rid in requests}
    for record in steps:
        out = outputs.get(record["step"])
        row = 0
        for entry in record["entries"]:
            for place in entry["want"]:
                rows[entry["id"]][pos[entry["id"]] + place] = out[row]
                row += 1
            pos[entry["id"]] += len(entry["tokens"])
    return {rid: torch.stack(r) for rid, r in rows.items()}


def peak_tokens(steps: list[dict], rounding: int = 64) -> int:
    """The most tokens live requests hold at any time, each rounded up to ``rounding``."""
    held: dict[str, int] = {}
    peak = 0
    for record in steps:
        for entry in record["entries"]:
            held[entry["id"]] = held.get(entry["id"], 0) + len(entry["tokens"])
        peak = max(peak, sum(-(-n // rounding) * rounding for n in held.values()))
        for rid in record["end"]:
            held.pop(rid, None)
    return peak
