"""Interfaces of the parts a model is put together from.

A model is data: an embedding, a list of layers, the order in which the layers run, a final
norm and a head.  Each layer names a block arrangement and, inside it, a mixer, a feed-forward
and norms, every one a :class:`PartSpec` (a registered kind plus its sizes and constants).
No part knows which architecture it serves; what a part needs it gets as constructor
parameters, as tensors by name, and as the :class:`StepContext` of the running step.

The reference hard-wires one block (src/turboserve/engine/model/layers.py:443-487) and one
cache kind (src/turboserve/engine/core/kv_cache.py:372-386); the split below is this engine's.
"""

from __future__ import annotations

from collections.abc import Mapping
from dataclasses import dataclass, field
from typing import TYPE_CHECKING, Any

import torch

if TYPE_CHECKING:  # pragma: no cover
    from turboserve_amd.engine.batch import StepContext


# ---------------------------------------------------------------------------------------------
# plain-data descriptions
# ---------------------------------------------------------------------------------------------


@dataclass(frozen=True)
class PartSpec:
    """A registered part ``kind`` and the keyword parameters it is built with."""

    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)


@dataclass(frozen=True)
class TensorSpec:
    """What a part expects under one checkpoint tensor name.

    ``kind`` is ``"float"`` (converted to the run's dtype), ``"float_keep32"`` (a tensor the
    file stores in 32-bit stays 32-bit, anything else is converted to the run's dtype) or
    ``"int"`` (kept as int32).  ``init`` says how the random-weights mode fills it:
    ``"normal"`` (N(0, std)), ``"ones"`` or ``"zeros"``.
    """

    shape: tuple[int, ...]
    kind: str = "float"
    init: str = "normal"


@dataclass(frozen=True)
class PagedKV:
    """A mixer's need for per-token cache pages: per token ``num_kv_heads`` keys of ``head_dim``
    elements and as many values of ``value_dim`` (``None``: as wide as the keys; 0: the mixer
    caches one vector per token and head, and the value pages have no room at all);
    ``window`` keys are ever read again (``None``: all of them)."""

    num_kv_heads: int
    head_dim: int
    window: int | None = None
    value_dim: int | None = None

    @property
    def value_width(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim


@dataclass(frozen=True)
class FixedState:
    """A mixer's need for per-request state of fixed size (``shape`` elements of ``dtype``
    per request), zeroed when a request takes its slot."""

    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


#: What a mixer asks of the cache: nothing, pages, fixed-size state, or several of these (a
#: layer that keeps pages and a state of its own gets one view for each, in the order asked).
CacheNeed = PagedKV | FixedState | None | tuple


@dataclass
class PagedKVView:
    """One cache unit's pages: ``k`` is ``[num_blocks, kv_heads, block_size, head_dim]``, ``v`` is
    stored transposed, ``[num_blocks, kv_heads, value_dim, block_size]`` (``value_dim`` is
    ``head_dim`` unless the mixer asked otherwise); ``group`` indexes the step's per-group block
    tables and slot mappings; ``writable`` is false when the layer reads another layer's cache."""

    k: torch.Tensor
    v: torch.Tensor
    group: int
    block_size: int
    window: int | None
    writable: bool = True


@dataclass
class FixedStateView:
    """One cache unit's per-request state: ``[num_slots, *shape]``; the rows of this step's
    requests are ``ctx.state_slots``."""

    state: torch.Tensor
    writable: bool = True


#: What a layer call is handed: the view of its one need, or a tuple of views, one per need.
CacheView = PagedKVView | FixedStateView | None | tuple


@dataclass
class Runtime:
    """What every part is built with: the device, the run's dtype and the kernel library.

    ``shared`` holds parts without weights that several layers may use as one object (the
    rotary tables: one per distinct set of constants, not one per layer)."""

    device: torch.device
    dtype: torch.dtype
    ops: Any  # turboserve_amd.kernels.ops.Ops
    shared: dict = field(default_factory=dict)


@dataclass
class ResidualStream:
    """The hidden state between blocks: a 32-bit running sum ``residual [T, H]`` and the last
    part's output ``pending [T, H]`` (run dtype) that has not been added to it yet."""

    residual: torch.Tensor
    pending: torch.Tensor | None = None  # [T, H] run dtype, or [S, T, H] 32-bit partial sums


# ---------------------------------------------------------------------------------------------
# interfaces
# ---------------------------------------------------------------------------------------------


class Part:
    """Base of everything that holds weights.

    ``prefix`` is the checkpoint name prefix of the part (``"model.layers.3.self_attn"``).
    ``tensor_specs`` maps full checkpoint names to what is expected there; ``load`` receives
    exactly those tensors, on the device, already converted, and may fuse or re-lay them.
    """

    #: A part without weights whose instances with equal parameters may be one object.
    shareable = False
    #: Whether a step through this part may be recorded into a HIP graph: it reads nothing back
    #: to the host (no ``.item()``, ``.tolist()``, ``nonzero()``) and what it launches depends only
    #: on the step's shape, not on device data.  A part that cannot promise this says False and
    #: the runner then runs every step of the model eagerly.
    capturable = True

    def __init__(self, prefix: str, runtime: Runtime) -> None:
        self.prefix = prefix
        self.runtime = runtime

    def name(self, suffix: str) -> str:
        return f"{self.prefix}.{suffix}" if self.prefix else suffix

    def is_capturable(self) -> bool:
        """``capturable`` of this part and of the parts it is made of."""
        return self.capturable

    def tensor_specs(self) -> dict[str, TensorSpec]:
        return {}

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:  # pragma: no cover - default
        return None

    def step_fields(self) -> tuple:
        """Integer fields this part wants in every step's packed buffer beside the engine's own
        (``engine.batch.StepField``: a name, a length rule, a function that fills it from the
        step's entries, a padding value): per-token, per-request or per-step numbers that the
        host knows and the part's kernels need on the device, in eager and in recorded steps
        alike.  The part finds them as ``ctx.extras[name]``."""
        return ()

    def activation_bytes(self, tokens: int, itemsize: int) -> int:
        """Bytes of the transient tensors this part holds at once in a step of ``tokens`` rows
        (``itemsize``: bytes of a run-dtype element).  The engine sums these over the model to
        leave room beside the cache pages; a part that makes nothing large may say 0."""
        return 0


class Norm(Part):
    """Normalisation over the last dimension."""

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """``[T, H]`` run dtype -> ``[T, H]`` run dtype."""
        raise NotImplementedError

    def forward_residual(self, stream: ResidualStream, rows: torch.Tensor | None = None) -> torch.Tensor:
        """Add ``stream.pending`` into ``stream.residual`` (32-bit) and return the normalised
        sum in the run dtype.  With ``rows`` only those rows are read and returned, and the
        stream is left as it is."""
        raise NotImplementedError


class PositionEncoding(Part):
    """Encodes positions into the queries and keys of an attention mixer and stores the
    step's keys and values into the cache pages (one pass over the projection output)."""

    def encode_and_store(
        self,
        qkv: torch.Tensor,
        num_heads: int,
        num_kv_heads: int,
        head_dim: int,
        ctx: "StepContext",
        cache: PagedKVView,
    ) -> tuple[torch.Tensor, int]:
        """``qkv``: the fused projection ``[T, (Hq + 2 Hkv) D]`` as ``ops.linear`` returned it (a
        tensor of the run dtype, or 32-bit partial sums ``[S, T, ..]``).  Encodes q and k, writes
        k, v at the step's slots of ``cache.group`` unless the cache is not writable, and
        returns the tensor holding the encoded queries with its row stride."""
        raise NotImplementedError

    def score_slopes(self, num_heads: int) -> torch.Tensor | None:
        """An encoding may (also, or instead) act inside the scores: ``[num_heads]`` 32-bit
        slopes ``m`` on the device, for which the score of key ``j`` for the query at position
        ``p`` of head ``h`` gets ``m[h] * (j - p)`` added before the softmax; ``None``: no such
        bias.  The attention mixer hands them to a kernel that takes them."""
        return None


class Embedding(Part):
    """Token ids -> what the first layer's residual stream starts as."""

    def forward(self, token_ids: torch.Tensor, ctx: "StepContext") -> torch.Tensor:
        """``token_ids [T]`` int32 -> 32-bit ``[T, H]``."""
        raise NotImplementedError


class Head(Part):
    """The residual stream after the last layer, at the rows whose scores are wanted -> 32-bit
    scores over the vocabulary.  A head that shares a tensor with another part (a tied head
    shares the embedding's table) names that tensor in its ``tensor_specs`` like any other."""

    def forward(self, stream: ResidualStream, rows: torch.Tensor) -> torch.Tensor:
        """``rows [n]`` int32 -> ``[n, V]`` 32-bit; the stream is left as it is."""
        raise NotImplementedError

    def ignorable_names(self) -> set[str]:
        """Tensor names a checkpoint may hold for this part that it does not read."""
        return set()


class Mixer(Part):
    """Mixes information between the tokens of a request (attention, or anything with state)."""

    def cache_need(self) -> CacheNeed:
        """``None``, one :class:`PagedKV` or :class:`FixedState`, or a tuple of them; ``forward``
        gets the matching view, or a tuple of views in the same order."""
        return None

    def forward(self, x: torch.Tensor, ctx: "StepContext", cache: CacheView) -> torch.Tensor:
        """``x [T, H]`` (normalised) -> ``[T, H]`` of the run dtype (or, straight from
        ``ops.linear``, ``[S, T, H]`` 32-bit partial sums).  The rows of request ``s`` are
        ``ctx.query_start_loc[s]:ctx.query_start_loc[s+1]``, in position order, continuing
        whatever earlier steps left in ``cache``."""
        raise NotImplementedError


class FeedForward(Part):
    """Acts on each token alone."""

    def forward(self, x: torch.Tensor, ctx: "StepContext") -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    """An arrangement of norms, a mixer and a feed-forward around the residual stream."""

    mixer: Mixer

    def forward(self, stream: ResidualStream, ctx: "StepContext", cache: CacheView) -> ResidualStream:
        raise NotImplementedError

    def is_capturable(self) -> bool:
        return self.capturable and all(part.is_capturable() for part in self.parts())

    def step_fields(self) -> tuple:
        return tuple(one for part in self.parts() for one in part.step_fields())

    def activation_bytes(self, tokens: int, itemsize: int) -> int:
        """The largest of its parts' needs: they run one after the other."""
        return max((part.activation_bytes(tokens, itemsize) for part in self.parts()), default=0)

    def parts(self) -> list[Part]:
        raise NotImplementedError
