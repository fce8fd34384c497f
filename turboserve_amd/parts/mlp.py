"""SwiGLU feed-forward (src/turboserve/engine/model/layers.py:394-440)."""

from __future__ import annotations

from collections.abc import Mapping

import torch

from turboserve_amd.parts.base import FeedForward, Runtime, TensorSpec
from turboserve_amd.parts.registry import register_feed_forward


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    """``down(silu(gate(x)) * up(x))`` (layers.py:437-440).  Gate and up are held as one
    ``[2 I, H]`` matrix whose rows alternate gate, up (interleaved at load; the checkpoint keeps
    them apart): a step does one product for both, and the product's kernel has each gate
    value next to its up value, so it can apply the activation itself."""

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

    def activation_bytes(self, tokens: int, itemsize: int) -> int:
        """The gate|up projection, the activated product and the down projection (32-bit: it is
        added to the residual stream) of a step."""
        return tokens * (3 * self.intermediate_size * itemsize + self.hidden_size * 4)

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        gate, up = tensors[self.name("gate_proj.weight")], tensors[self.name("up_proj.weight")]
        self.gate_up_weight = torch.stack([gate, up], dim=1).reshape(2 * gate.shape[0], gate.shape[1]).contiguous()
        self.down_weight = tensors[self.name("down_proj.weight")].contiguous()

    def forward(self, x: torch.Tensor, ctx) -> torch.Tensor:
        ops = self.runtime.ops
        return ops.linear(ops.linear_swiglu(x, self.gate_up_weight), self.down_weight, for_residual=True)
