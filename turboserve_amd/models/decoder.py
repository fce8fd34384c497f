"""A decoder assembled from a plan: embedding, layers, the order they run in, final norm, head.

The plan is data.  ``layers`` describes each layer's block and parts; ``schedule`` is the list
of layer calls of one forward pass: it may name a layer twice (the layer's weights run twice,
each call with a cache of its own) and a call may read the cache of an earlier call instead of
owning one.  The reference runs its layers once each, in order, with one cache kind
(src/turboserve/engine/model/model.py:82-108); a plan with ``schedule = [0, 1, .. L-1]`` is
that.
"""

from __future__ import annotations

from collections.abc import Mapping, Sequence
from dataclasses import dataclass

import torch

from turboserve_amd.parts.base import (
    Block,
    CacheNeed,
    CacheView,
    PartSpec,
    ResidualStream,
    Runtime,
    TensorSpec,
)
from turboserve_amd.parts.registry import build_part


@dataclass(frozen=True)
class LayerSpec:
    """One layer: the checkpoint prefix of its tensors and its block (kind + parts)."""

    prefix: str
    block: PartSpec


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order: which layer runs and, optionally, the index of an EARLIER
    entry whose cache it reads (it then writes nothing)."""

    layer: int
    cache_of: int | None = None


@dataclass(frozen=True)
class ModelPlan:
    vocab_size: int
    hidden_size: int
    layers: tuple[LayerSpec, ...]
    schedule: tuple[LayerCall, ...]
    final_norm: PartSpec
    tie_head: bool
    embedding_name: str = "model.embed_tokens"
    final_norm_name: str = "model.norm"
    head_name: str = "lm_head"

    def __post_init__(self) -> None:
        for index, call in enumerate(self.schedule):
            if not 0 <= call.layer < len(self.layers):
                raise ValueError(f"schedule entry {index} names layer {call.layer} of {len(self.layers)}")
            if call.cache_of is not None:
                if not 0 <= call.cache_of < index:
                    raise ValueError(f"schedule entry {index} reads the cache of entry {call.cache_of}, which is not earlier")
                if self.schedule[call.cache_of].cache_of is not None:
                    raise ValueError(f"schedule entry {index} reads the cache of entry {call.cache_of}, which owns none")


class DecoderModel:
    """The model object the step function drives.  It owns weights, not caches: the caches of
    a step come in as one view per schedule entry."""

    def __init__(self, plan: ModelPlan, runtime: Runtime) -> None:
        self.plan = plan
        self.runtime = runtime
        self.blocks: list[Block] = [
            build_part("block", layer.block, layer.prefix, runtime) for layer in plan.layers
        ]
        self.final_norm = build_part("norm", plan.final_norm, plan.final_norm_name, runtime)
        self.embedding: torch.Tensor | None = None
        self.head: torch.Tensor | None = None

    # -- weights ------------------------------------------------------------------------------

    def tensor_specs(self) -> dict[str, TensorSpec]:
        """Every checkpoint tensor the model expects, in model order."""
        plan = self.plan
        specs: dict[str, TensorSpec] = {
            f"{plan.embedding_name}.weight": TensorSpec((plan.vocab_size, plan.hidden_size))
        }
        for block in self.blocks:
            specs.update(block.tensor_specs())
        specs.update(self.final_norm.tensor_specs())
        if not plan.tie_head:
            specs[f"{plan.head_name}.weight"] = TensorSpec((plan.vocab_size, plan.hidden_size))
        return specs

    def ignorable_names(self) -> set[str]:
        """Names a checkpoint may hold that the model does not read: a tied model's copy of the
        head (the reference shares one parameter, src/turboserve/engine/model/model.py:139-142)."""
        return {f"{self.plan.head_name}.weight"} if self.plan.tie_head else set()

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        plan = self.plan
        self.embedding = tensors[f"{plan.embedding_name}.weight"].contiguous()
        for block in self.blocks:
            block.load(tensors)
        self.final_norm.load(tensors)
        self.head = self.embedding if plan.tie_head else tensors[f"{plan.head_name}.weight"].contiguous()

    def num_parameters(self) -> int:
        total = 0
        for spec in self.tensor_specs().values():
            count = 1
            for dim in spec.shape:
                count *= dim
            total += count
        return total

    def activation_bytes(self, tokens: int, requests: int, itemsize: int) -> int:
        """Room a step of ``tokens`` rows that wants logits for ``requests`` of them takes beside
        weights and cache: the 32-bit residual stream and the output waiting to be added to it,
        the neediest layer (norm output plus its largest part), twice over because the caching
        allocator keeps freed blocks of other sizes, and the 32-bit logits with the sampler's
        working copy (the reference's estimate has the same terms from Qwen2's sizes,
        src/turboserve/engine/runtime/memory.py:208-242)."""
        plan = self.plan
        stream = tokens * plan.hidden_size * (4 + 4)
        layer = max((block.activation_bytes(tokens, itemsize) for block in self.blocks), default=0)
        layer += self.final_norm.activation_bytes(tokens, itemsize)
        return 2 * (stream + layer) + requests * plan.vocab_size * 4 * 2

    # -- caches -------------------------------------------------------------------------------

    def is_capturable(self) -> bool:
        """Whether single-token steps of this model may be recorded into HIP graphs: every
        part says so (``Part.capturable``)."""
        return all(block.is_capturable() for block in self.blocks) and self.final_norm.is_capturable()

    def cache_needs(self) -> list[CacheNeed]:
        """What each schedule entry needs a cache for (``None``: nothing, or it reads another's)."""
        needs: list[CacheNeed] = []
        for call in self.plan.schedule:
            need = self.blocks[call.layer].mixer.cache_need()
            needs.append(None if call.cache_of is not None else need)
        return needs

    # -- the pass -----------------------------------------------------------------------------

    def forward(self, token_ids: torch.Tensor, ctx, caches: Sequence[CacheView]) -> ResidualStream:
        """Embedding and every scheduled layer call over the step's flat tokens
        (model.py:105-107).  ``caches[i]`` is the view of schedule entry ``i``."""
        if len(caches) != len(self.plan.schedule):
            raise ValueError(f"{len(caches)} cache views for {len(self.plan.schedule)} scheduled layer calls")
        stream = ResidualStream(self.runtime.ops.embed(self.embedding, token_ids))
        for call, cache in zip(self.plan.schedule, caches):
            stream = self.blocks[call.layer].forward(stream, ctx, cache)
        return stream

    def logits(self, stream: ResidualStream, rows: torch.Tensor) -> torch.Tensor:
        """Final norm and head at ``rows`` only -> 32-bit ``[n, V]`` (model.py:108, 237-244)."""
        hidden = self.final_norm.forward_residual(stream, rows)
        return self.runtime.ops.linear_float32_out(hidden, self.head)
