"""SwiGLU feed-forward (src/turboserve/engine/model/layers.py:394-440)."""

from __future__ import annotations

from collections.abc import Mapping

import torch

from turboserve_amd.parts.base import FeedForward, Runtime, TensorSpec
from turboserve_amd.parts.registry import register_feed_forward


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    """``down(silu(gate(x)) * up(x))`` (layers.py:437-440).  Gate and up are held as one
    ``[2 I, H]`` matrix (concatenated at load), so a step does one product for both."""

    def __init__(self, prefix: str, runtime: Runtime, *, hidden_size: int, intermediate_size: int) -> None:
        super().__init__(prefix, runtime)
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.gate_up_weight: torch.Tensor | None = None
        self.down_weight: torch.Tensor | None = None

    def tensor_specs(self) -> dict[str, TensorSpec]:
        return {
            self.name("gate_proj.weight"): TensorSpec((self.intermediate_size, self.hidden_size)),
            self.name("up_proj.weight"): TensorSpec((self.intermediate_size, self.hidden_size)),
            self.name("down_proj.weight"): TensorSpec((self.hidden_size, self.intermediate_size)),
        }

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.gate_up_weight = torch.cat(
            [tensors[self.name("gate_proj.weight")], tensors[self.name("up_proj.weight")]], dim=0
        ).contiguous()
        self.down_weight = tensors[self.name("down_proj.weight")].contiguous()

    def forward(self, x: torch.Tensor, ctx) -> torch.Tensor:
        ops = self.runtime.ops
        gate_up = ops.linear(x, self.gate_up_weight)
        return ops.linear(ops.swiglu(gate_up, self.runtime.dtype), self.down_weight)
