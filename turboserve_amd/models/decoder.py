"""A decoder assembled from a plan: embedding, layers, the order they run in, head.

The plan is data.  ``embedding`` and ``head`` are parts like any other (for the usual pair see
``parts.ends.standard_ends``); ``layers`` describes each layer's block and parts; ``schedule`` is the list
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
    Embedding,
    Head,
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
    embedding: PartSpec
    head: PartSpec
    embedding_prefix: str = "model.embed_tokens"
    head_prefix: str = "lm_head"

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
        self.embedding: Embedding = build_part("embedding", plan.embedding, plan.embedding_prefix, runtime)
        self.head: Head = build_part("head", plan.head, plan.head_prefix, runtime)

    # -- weights ------------------------------------------------------------------------------

    def tensor_specs(self) -> dict[str, TensorSpec]:
        """Every checkpoint tensor the model expects, in model order."""
        specs: dict[str, TensorSpec] = dict(self.embedding.tensor_specs())
        for block in self.blocks:
            specs.update(block.tensor_specs())
        for name, spec in self.head.tensor_specs().items():
            # A head may name a tensor of another part (a tied head: the token table) and then
            # shares it; both must expect the same thing there.
            if name in specs and specs[name] != spec:
                raise ValueError(f"the head expects {spec} under {name!r}, another part {specs[name]}")
            specs[name] = spec
        return specs

    def ignorable_names(self) -> set[str]:
        """Names a checkpoint may hold that the model does not read (a tied head's own copy of
        the matrix)."""
        return self.head.ignorable_names()

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.embedding.load(tensors)
        for block in self.blocks:
            block.load(tensors)
        self.head.load(tensors)

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
        layer += self.head.activation_bytes(tokens, itemsize)
        return 2 * (stream + layer) + requests * plan.vocab_size * 4 * 2

    # -- caches -------------------------------------------------------------------------------

    def is_capturable(self) -> bool:
        """Whether single-token steps of this model may be recorded into HIP graphs: every
        part says so (``Part.capturable``)."""
        return (all(block.is_capturable() for block in self.blocks) and self.embedding.is_capturable()
                and self.head.is_capturable())

    def step_fields(self) -> tuple:
        """The integer fields the model's parts want in every step's packed buffer beside the
        engine's own (``Part.step_fields``), each name once."""
        from turboserve_amd.engine.batch import merge_step_fields

        asked = [*self.embedding.step_fields()]
        for block in self.blocks:
            asked.extend(block.step_fields())
        asked.extend(self.head.step_fields())
        return merge_step_fields(asked)

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
        stream = ResidualStream(self.embedding.forward(token_ids, ctx))
        for call, cache in zip(self.plan.schedule, caches):
            stream = self.blocks[call.layer].forward(stream, ctx, cache)
        return stream

    def logits(self, stream: ResidualStream, rows: torch.Tensor) -> torch.Tensor:
        """The head at ``rows`` only -> 32-bit ``[n, V]`` (model.py:108, 237-244)."""
        return self.head.forward(stream, rows)
