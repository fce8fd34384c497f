"""Rotary position encoding (src/turboserve/engine/model/layers.py:214-308)."""

from __future__ import annotations

import torch

from turboserve_amd.parts.base import PagedKVView, PositionEncoding, Runtime
from turboserve_amd.parts.registry import register_position_encoding


def rotary_tables(capacity: int, head_dim: int, theta: float, factor: float) -> tuple[torch.Tensor, torch.Tensor]:
    """32-bit ``cos, sin [capacity, D/2]`` of the angles ``(pos / factor) * theta^(-2i/D)``.

    Computed on the CPU with the reference's expressions (layers.py:258-262 for the inverse
    frequencies, :281-286 for the outer product; its tables repeat the ``D/2`` columns twice,
    which is not stored here)."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    positions = torch.arange(capacity, dtype=torch.float32)
    if factor != 1.0:
        positions = positions / factor
    angles = torch.outer(positions, inv_freq)
    return angles.cos().contiguous(), angles.sin().contiguous()


@register_position_encoding("rope")
class RotaryEncoding(PositionEncoding):
    """Half-split rotary encoding: the pair ``(i, i + D/2)`` of every query and key head is
    turned by the angle of the token's position (layers.py:214-222, 298-302).  The rotation is
    computed in 32-bit from 32-bit tables and rounded once.  It has no weights, so layers with
    the same constants share one instance and one pair of tables.

    The tables are made once, at the first step, for ``max_positions`` (the model's
    ``max_position_embeddings``) or ``initial_positions`` when given; a step that reaches
    further makes them grow by doubling, driven by the host-known largest position
    (layers.py:272-288).  A recorded step (a HIP graph) holds the addresses of the tables it was
    recorded with, so tables that growth has superseded are kept, never freed: they cover every
    position such a recording can bring, because the recording's widest context was inside them
    when it was made."""

    shareable = True

    def __init__(
        self,
        prefix: str,
        runtime: Runtime,
        *,
        head_dim: int,
        theta: float,
        scaling_factor: float = 1.0,
        max_positions: int = 2048,
        initial_positions: int | None = None,
    ) -> None:
        super().__init__(prefix, runtime)
        if head_dim % 2 != 0:
            raise ValueError(f"head_dim must be even for rotary encoding, got {head_dim}")
        self.head_dim = int(head_dim)
        self.theta = float(theta)
        self.scaling_factor = float(scaling_factor)
        self.cos: torch.Tensor | None = None
        self.sin: torch.Tensor | None = None
        self.capacity = 0
        #: First table size; the tables themselves are made at the first step.  The reference
        #: starts at ``min(max_positions, 1024)`` (layers.py:265); here the whole of
        #: ``max_positions`` is made at once (7B: 32,768 x 64 x 4 bytes x 2 = 16.8 MB), so that
        #: growth is the exception.
        self.initial_capacity = int(max_positions if initial_positions is None else initial_positions)
        #: Tables that growth has replaced; recorded steps may still read them.
        self.superseded: list[tuple[torch.Tensor, torch.Tensor]] = []

    def ensure_capacity(self, num_positions: int) -> None:
        if num_positions <= self.capacity:
            return
        target = max(num_positions, 2 * self.capacity, self.initial_capacity, 16)
        cos, sin = rotary_tables(target, self.head_dim, self.theta, self.scaling_factor)
        if self.cos is not None:
            self.superseded.append((self.cos, self.sin))
        self.cos = cos.to(self.runtime.device)
        self.sin = sin.to(self.runtime.device)
        self.capacity = target

    def encode_and_store(self, qkv, num_heads, num_kv_heads, head_dim, ctx, cache: PagedKVView):
        self.ensure_capacity(ctx.max_context_len)
        slots = ctx.slot_mapping[cache.group] if cache.writable else None
        return self.runtime.ops.rope_store(
            qkv, cache.k, cache.v, self.cos, self.sin, ctx.positions, slots,
            num_heads, num_kv_heads, head_dim, cache.block_size, ctx.max_context_len - 1, self.runtime.dtype,
        )


@register_position_encoding("none")
class NoPositionEncoding(PositionEncoding):
    """No encoding: queries and keys stay as projected; keys and values are stored."""

    shareable = True

    def __init__(self, prefix: str, runtime: Runtime) -> None:
        super().__init__(prefix, runtime)

    def encode_and_store(self, qkv, num_heads, num_kv_heads, head_dim, ctx, cache: PagedKVView):
        slots = ctx.slot_mapping[cache.group] if cache.writable else None
        return self.runtime.ops.rope_store(
            qkv, cache.k, cache.v, None, None, ctx.positions, slots,
            num_heads, num_kv_heads, head_dim, cache.block_size, ctx.max_context_len - 1, self.runtime.dtype,
        )
