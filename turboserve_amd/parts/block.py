"""Block arrangements (src/turboserve/engine/model/layers.py:443-487)."""

from __future__ import annotations

from collections.abc import Mapping

import torch

from turboserve_amd.parts.base import Block, CacheView, Part, PartSpec, ResidualStream, Runtime, TensorSpec
from turboserve_amd.parts.registry import build_part, register_block


@register_block("prenorm")
class PreNormBlock(Block):
    """``h += mixer(norm_a(h)); h += feed_forward(norm_b(h))`` (layers.py:479-487).

    The sums are carried in the 32-bit residual stream; each part's output waits in
    ``stream.pending`` until the next norm adds it, in the same pass that normalises.
    ``mixer_norm_name`` / ``ff_norm_name`` / ``mixer_name`` / ``ff_name`` are the checkpoint
    names of the four parts under the block's prefix."""

    def __init__(
        self,
        prefix: str,
        runtime: Runtime,
        *,
        mixer: PartSpec,
        feed_forward: PartSpec,
        mixer_norm: PartSpec,
        ff_norm: PartSpec,
        mixer_name: str = "self_attn",
        ff_name: str = "mlp",
        mixer_norm_name: str = "input_layernorm",
        ff_norm_name: str = "post_attention_layernorm",
    ) -> None:
        super().__init__(prefix, runtime)
        self.mixer_norm = build_part("norm", mixer_norm, self.name(mixer_norm_name), runtime)
        self.mixer = build_part("mixer", mixer, self.name(mixer_name), runtime)
        self.ff_norm = build_part("norm", ff_norm, self.name(ff_norm_name), runtime)
        self.feed_forward = build_part("feed_forward", feed_forward, self.name(ff_name), runtime)

    def parts(self) -> list[Part]:
        return [self.mixer_norm, self.mixer, self.ff_norm, self.feed_forward]

    def activation_bytes(self, tokens: int, itemsize: int) -> int:
        """A norm's output stays alive while the part it feeds runs."""
        return max(
            self.mixer_norm.activation_bytes(tokens, itemsize) + self.mixer.activation_bytes(tokens, itemsize),
            self.ff_norm.activation_bytes(tokens, itemsize) + self.feed_forward.activation_bytes(tokens, itemsize),
        )

    def tensor_specs(self) -> dict[str, TensorSpec]:
        specs: dict[str, TensorSpec] = {}
        for part in self.parts():
            specs.update(part.tensor_specs())
        return specs

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        for part in self.parts():
            part.load(tensors)

    def forward(self, stream: ResidualStream, ctx, cache: CacheView) -> ResidualStream:
        x = self.mixer_norm.forward_residual(stream)
        stream.pending = self.mixer.forward(x, ctx, cache)
        x = self.ff_norm.forward_residual(stream)
        stream.pending = self.feed_forward.forward(x, ctx)
        return stream
