"""Where a step's time goes, from a ``rocprofv3 --kernel-trace`` CSV.

The reference embeds its hardware record in every result (src/turboserve/hwinfo.py:160-193) and
has no kernel-level measurement; this is this engine's.  A trace of a run holds set-up work
(weights being drawn, graphs being recorded) before the steps of interest, so the summary is
made over the LAST ``steps`` steps of the trace: a step ends with the kernel named by
``marker`` (by default the second stage of the greedy sampler, which every step of a greedy
run ends with).  Kernels are grouped by name and launch grid, since one kernel serves several
products of different sizes.

    rocprofv3 --kernel-trace --output-format csv -d OUT -- python bench.py ...
    python bench.py --kernel-shares OUT/<host>/<pid>_kernel_trace.csv [--shares-steps 4]
"""

from __future__ import annotations

import csv
import re
from collections import OrderedDict
from dataclasses import dataclass
from pathlib import Path

DEFAULT_MARKER = "argmax_rows_kernel"


@dataclass
class KernelShare:
    name: str
    grid: tuple[int, int, int]
    calls_per_step: float
    average_us: float
    per_step_us: float
    share: float


@dataclass
class StepShares:
    steps: int
    kernels_per_step: float
    span_us: float  # first kernel's start to last kernel's end, per step
    busy_us: float  # sum of kernel durations, per step
    rows: list[KernelShare]


def short_name(name: str) -> str:
    """A kernel's name without its return type, argument list and namespaces of libraries."""
    name = re.sub(r"^void\s+", "", name.strip()).replace("(anonymous namespace)::", "")
    depth, cut = 0, len(name)
    for index, char in enumerate(name):
        if char == "<":
            depth += 1
        elif char == ">":
            depth -= 1
        elif char == "(" and depth == 0:
            cut = index
            break
    name = name[:cut]
    if len(name) > 80:
        name = name[:77] + "..."
    return name


def read_trace(path: str | Path) -> list[dict]:
    """The kernel dispatches of a trace in start order: name, grid, start and end in ns."""
    rows = []
    with open(path, newline="", encoding="utf-8") as handle:
        for record in csv.DictReader(handle):
            if record.get("Kind", "KERNEL_DISPATCH") != "KERNEL_DISPATCH":
                continue
            rows.append({
                "name": record["Kernel_Name"],
                "grid": (int(record["Grid_Size_X"]), int(record["Grid_Size_Y"]), int(record["Grid_Size_Z"])),
                "start": int(record["Start_Timestamp"]),
                "end": int(record["End_Timestamp"]),
            })
    rows.sort(key=lambda row: row["start"])
    return rows


def step_shares(path: str | Path, *, steps: int = 4, marker: str = DEFAULT_MARKER) -> StepShares:
    """Per-kernel time of the last ``steps`` steps of the trace, averaged per step."""
    rows = read_trace(path)
    ends = [index for index, row in enumerate(rows) if marker in row["name"]]
    if len(ends) < steps + 1:
        raise ValueError(f"the trace holds {len(ends)} kernels named {marker!r}: not enough for {steps} whole steps")
    first, last = ends[-steps - 1] + 1, ends[-1]
    window = rows[first:last + 1]
    groups: "OrderedDict[tuple, list[int]]" = OrderedDict()
    for row in window:
        groups.setdefault((short_name(row["name"]), row["grid"]), []).append(row["end"] - row["start"])
    busy = sum(sum(durations) for durations in groups.values())
    shares = [
        KernelShare(name, grid, len(durations) / steps, sum(durations) / len(durations) / 1e3,
                    sum(durations) / steps / 1e3, sum(durations) / busy)
        for (name, grid), durations in groups.items()
    ]
    shares.sort(key=lambda share: -share.per_step_us)
    # Steps follow each other without a gap when they are launched ahead, so the span is taken
    # over the whole window and divided.
    span = (window[-1]["end"] - window[0]["start"]) / steps / 1e3
    return StepShares(steps, len(window) / steps, span, busy / steps / 1e3, shares)


def format_shares(result: StepShares, *, top: int = 16) -> str:
    """A Markdown table of the ``top`` groups and one line for the rest."""
    lines = [
        f"last {result.steps} steps of the trace: {result.kernels_per_step:.0f} kernels a step, "
        f"span {result.span_us:,.0f} us a step, kernels busy {result.busy_us:,.0f} us a step",
        "",
        "| kernel | grid (threads x, y, z) | calls a step | avg us | us a step | share |",
        "| --- | --- | --- | --- | --- | --- |",
    ]
    for share in result.rows[:top]:
        lines.append(f"| `{share.name}` | {share.grid[0]}, {share.grid[1]}, {share.grid[2]} | {share.calls_per_step:g} | "
                     f"{share.average_us:.1f} | {share.per_step_us:,.1f} | {100 * share.share:.1f}% |")
    rest = result.rows[top:]
    if rest:
        lines.append(f"| {len(rest)} other kernels | | {sum(s.calls_per_step for s in rest):g} | | "
                     f"{sum(s.per_step_us for s in rest):,.1f} | {100 * sum(s.share for s in rest):.1f}% |")
    return "\n".join(lines)
