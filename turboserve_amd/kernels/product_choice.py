"""Which kernel computes a bfloat16 projection of 17 to 64 rows: measured per shape.

Up to 16 rows the engine's weight-streaming product with resident activations is the fastest
kernel for every shape of this model family; above 64 rows the BLAS library behind ``torch.mm``
runs the projections, as in the reference (src/turboserve/engine/model/layers.py:142).  In
between neither wins everywhere: the engine's kernel is ahead for the products with a long inner
dimension or a short output (down, qkv, o), the library for a very wide output (gate|up, the
head at 64 rows).  So the choice is made by timing both on the model's own weights, once, at
start-up, for the two row counts the recorded decode steps use (32 and 64; other row counts take
the choice of the next power of two).

A library product chosen here is also recorded into the decode graphs.  Library kernels may
clear work space with a memset node, which has not replayed reliably on this hardware, so
before a shape is given to the library its product is recorded into a graph of its own and
replayed several times, with eager work in between, against the eager result; a shape that
fails stays with the engine's kernel.
"""

from __future__ import annotations

import logging
from collections.abc import Callable, Sequence
from dataclasses import dataclass

import torch

logger = logging.getLogger(__name__)

#: Row counts that are measured: the batch sizes of the recorded decode steps above 16.
MEASURED_ROWS = (32, 64)


def product_bucket(rows: int) -> int:
    """The measured row count whose choice ``rows`` takes."""
    return 1 if rows <= 1 else 1 << (rows - 1).bit_length()


@dataclass(frozen=True)
class ProductTiming:
    rows: int
    out_features: int
    in_features: int
    float32_out: bool
    own_us: float
    library_us: float
    library_verified: bool  # recorded into a graph and replayed exactly (only tried where it is faster)

    @property
    def library_chosen(self) -> bool:
        return self.library_verified and self.library_us < 0.97 * self.own_us


def _library(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, float32_out: bool) -> torch.Tensor:
    if float32_out:
        return torch.mm(x, weight.t(), out_dtype=torch.float32)
    return torch.mm(x, weight.t()) if bias is None else torch.addmm(bias, x, weight.t())


def _own(ops, x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, float32_out: bool) -> torch.Tensor:
    if float32_out:
        return ops.gemm_skinny(x, weight, max_splits=1)[0]
    return ops.gemm_skinny(x, weight, bias)


def _time_us(call: Callable[[int], object], operands: int, min_calls: int = 12) -> float:
    """Mean microseconds of ``call(i)`` over whole turns through the ``operands`` (the weights of
    the model's layers, so that every call streams its matrix from memory as a step does)."""
    turns = max(1, -(-min_calls // operands))
    for i in range(operands):
        call(i)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(turns):
        for i in range(operands):
            call(i)
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) * 1e3 / (turns * operands)


def library_product_replays(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None,
                            float32_out: bool, replays: int = 3) -> bool:
    """Whether the library's product for these operands, recorded into a HIP graph, gives the
    eager result bit for bit on every one of several replays with other work between them."""
    static_x = x.clone()
    _library(static_x, weight, bias, float32_out)  # the library's set-up happens outside the recording
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        recorded = _library(static_x, weight, bias, float32_out)
    generator = torch.Generator(device=x.device).manual_seed(7)
    for _ in range(replays):
        fresh = torch.randn(x.shape, device=x.device, dtype=torch.float32, generator=generator).to(x.dtype)
        static_x.copy_(fresh)
        eager = _library(static_x, weight, bias, float32_out)
        (eager.float() * 2.0).sum()  # unrelated eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        if not torch.equal(recorded, eager):
            return False
    return True


def choose_products(ops, run_step: Callable[[int], None], rows: Sequence[int] = MEASURED_ROWS) -> list[ProductTiming]:
    """Time the engine's kernel against the library for every projection shape that
    ``run_step(m)`` (a step over ``m`` rows, logits wanted at all of them) runs, for each ``m`` of
    ``rows``, and leave the choices in ``ops.library_products``.  Returns what was measured."""
    timings: list[ProductTiming] = []
    for m in rows:
        if not ops.skinny_resident_rows < m <= ops.skinny_max_rows or product_bucket(m) != m:
            raise ValueError(f"products are chosen at powers of two above {ops.skinny_resident_rows} "
                             f"up to {ops.skinny_max_rows} rows, got {m}")
        ops.product_log = []
        try:
            run_step(m)
        finally:
            seen, ops.product_log = ops.product_log, None
        shapes: dict[tuple, list[tuple[torch.Tensor, torch.Tensor | None]]] = {}
        for key, weight, bias in seen:
            held = shapes.setdefault(key, [])
            if all(weight.data_ptr() != other.data_ptr() for other, _ in held):
                held.append((weight, bias))
        for key, operands in shapes.items():
            _, n, k, _, float32_out = key
            x = (torch.randn((m, k), device=operands[0][0].device, dtype=torch.float32) * 0.5).to(torch.bfloat16)
            own_us = _time_us(lambda i: _own(ops, x, *operands[i], float32_out), len(operands))
            library_us = _time_us(lambda i: _library(x, *operands[i], float32_out), len(operands))
            verified = library_us < 0.97 * own_us and library_product_replays(x, *operands[0], float32_out)
            timing = ProductTiming(m, n, k, float32_out, own_us, library_us, verified)
            timings.append(timing)
            ops.library_products[key] = timing.library_chosen
            logger.info("product [%d, %d] x [%d, %d]%s: own kernel %.1f us, library %.1f us -> %s",
                        m, k, n, k, " (32-bit result)" if float32_out else "", own_us, library_us,
                        "library" if timing.library_chosen else "own kernel")
    return timings
