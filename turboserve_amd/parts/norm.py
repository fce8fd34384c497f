"""RMSNorm (src/turboserve/engine/model/layers.py:178-211)."""

from __future__ import annotations

from collections.abc import Mapping

import torch

from turboserve_amd.parts.base import Norm, ResidualStream, Runtime, TensorSpec
from turboserve_amd.parts.registry import register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    """``weight * round(x * rsqrt(mean(x^2) + eps))``: statistics in 32-bit, the normalised
    value rounded to the run dtype before the gain (layers.py:202-208).  The fused form also
    carries the residual sum, kept in 32-bit."""

    def __init__(self, prefix: str, runtime: Runtime, *, size: int, eps: float) -> None:
        super().__init__(prefix, runtime)
        self.size = int(size)
        self.eps = float(eps)
        self.weight: torch.Tensor | None = None

    def tensor_specs(self) -> dict[str, TensorSpec]:
        return {self.name("weight"): TensorSpec((self.size,), init="ones")}

    def activation_bytes(self, tokens: int, itemsize: int) -> int:
        return tokens * self.size * itemsize

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.weight = tensors[self.name("weight")].contiguous()

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.runtime.ops.rmsnorm(x, self.weight, self.eps)

    def forward_residual(self, stream: ResidualStream, rows: torch.Tensor | None = None) -> torch.Tensor:
        y = self.runtime.ops.add_rmsnorm(stream.residual, stream.pending, self.weight, self.eps, rows)
        if rows is None:
            stream.pending = None
        return y
