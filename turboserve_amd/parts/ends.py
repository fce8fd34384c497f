"""The two ends of a decoder: the token table its residual stream starts from, and the head
that turns the stream into scores over the vocabulary (src/turboserve/engine/model/model.py:
64-72 and :105-108, :139-142 for the tie)."""

from __future__ import annotations

from collections.abc import Mapping

import torch

from turboserve_amd.parts.base import Embedding, Head, PartSpec, ResidualStream, Runtime, TensorSpec
from turboserve_amd.parts.registry import build_part, register_embedding, register_head


@register_embedding("token_table")
class TokenTable(Embedding):
    """One row of ``[V, H]`` per token id, into the 32-bit residual stream."""

    def __init__(self, prefix: str, runtime: Runtime, *, vocab_size: int, hidden_size: int) -> None:
        super().__init__(prefix, runtime)
        self.vocab_size = int(vocab_size)
        self.hidden_size = int(hidden_size)
        self.weight: torch.Tensor | None = None

    def tensor_specs(self) -> dict[str, TensorSpec]:
        return {self.name("weight"): TensorSpec((self.vocab_size, self.hidden_size))}

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.weight = tensors[self.name("weight")].contiguous()

    def forward(self, token_ids: torch.Tensor, ctx) -> torch.Tensor:
        return self.runtime.ops.embed(self.weight, token_ids)


@register_head("norm_linear")
class NormLinearHead(Head):
    """A norm over the summed stream, then ``[V, H]`` without bias, at the wanted rows only
    (model.py:108, :237-244).  ``tied_to`` names the tensor of another part (the token table)
    that serves as the matrix; the checkpoint's own copy under this part's prefix is then not
    read (the reference shares one parameter, model.py:139-142)."""

    def __init__(
        self,
        prefix: str,
        runtime: Runtime,
        *,
        vocab_size: int,
        hidden_size: int,
        norm: PartSpec,
        norm_prefix: str,
        tied_to: str | None,
    ) -> None:
        super().__init__(prefix, runtime)
        self.vocab_size = int(vocab_size)
        self.hidden_size = int(hidden_size)
        self.norm = build_part("norm", norm, norm_prefix, runtime)
        self.tied_to = tied_to
        self.weight: torch.Tensor | None = None

    @property
    def weight_name(self) -> str:
        return self.tied_to or self.name("weight")

    def is_capturable(self) -> bool:
        return self.capturable and self.norm.is_capturable()

    def tensor_specs(self) -> dict[str, TensorSpec]:
        specs = dict(self.norm.tensor_specs())
        specs[self.weight_name] = TensorSpec((self.vocab_size, self.hidden_size))
        return specs

    def ignorable_names(self) -> set[str]:
        return {self.name("weight")} if self.tied_to else set()

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.norm.load(tensors)
        self.weight = tensors[self.weight_name].contiguous()

    def activation_bytes(self, tokens: int, itemsize: int) -> int:
        return self.norm.activation_bytes(tokens, itemsize)

    def forward(self, stream: ResidualStream, rows: torch.Tensor) -> torch.Tensor:
        hidden = self.norm.forward_residual(stream, rows)
        return self.runtime.ops.linear_float32_out(hidden, self.weight)


def standard_ends(vocab_size: int, hidden_size: int, norm: PartSpec, *, tie_head: bool,
                  embedding_prefix: str = "model.embed_tokens", norm_prefix: str = "model.norm") -> dict:
    """The ``embedding`` and ``head`` entries of a plan for the usual pair: a token table, and a
    final norm followed by a matrix that is the table itself (``tie_head``) or the head's own."""
    return {
        "embedding": PartSpec("token_table", {"vocab_size": vocab_size, "hidden_size": hidden_size}),
        "head": PartSpec("norm_linear", {
            "vocab_size": vocab_size, "hidden_size": hidden_size, "norm": norm, "norm_prefix": norm_prefix,
            "tied_to": f"{embedding_prefix}.weight" if tie_head else None,
        }),
        "embedding_prefix": embedding_prefix,
    }
