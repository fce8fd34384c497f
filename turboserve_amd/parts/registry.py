"""Registries from a part's kind name to its class, one per interface.

A layer description names its parts by kind, and so does a model for its embedding and its
head; adding a mixer, feed-forward, norm, position encoding, block arrangement, embedding or head
is one ``register_*`` call and needs no change elsewhere.
"""

from __future__ import annotations

from collections.abc import Callable
from typing import Any, TypeVar

from turboserve_amd.parts.base import PartSpec, Runtime

T = TypeVar("T")

MIXERS: dict[str, type] = {}
FEED_FORWARDS: dict[str, type] = {}
NORMS: dict[str, type] = {}
POSITION_ENCODINGS: dict[str, type] = {}
BLOCKS: dict[str, type] = {}
EMBEDDINGS: dict[str, type] = {}
HEADS: dict[str, type] = {}

_TABLES = {
    "mixer": MIXERS,
    "feed_forward": FEED_FORWARDS,
    "norm": NORMS,
    "position_encoding": POSITION_ENCODINGS,
    "block": BLOCKS,
    "embedding": EMBEDDINGS,
    "head": HEADS,
}


def _register(table: dict[str, type], role: str, kind: str) -> Callable[[type[T]], type[T]]:
    def decorate(cls: type[T]) -> type[T]:
        if kind in table and table[kind] is not cls:
            raise ValueError(f"{role} kind {kind!r} is already registered to {table[kind].__name__}")
        table[kind] = cls
        return cls

    return decorate


def register_mixer(kind: str) -> Callable[[type[T]], type[T]]:
    return _register(MIXERS, "mixer", kind)


def register_feed_forward(kind: str) -> Callable[[type[T]], type[T]]:
    return _register(FEED_FORWARDS, "feed_forward", kind)


def register_norm(kind: str) -> Callable[[type[T]], type[T]]:
    return _register(NORMS, "norm", kind)


def register_position_encoding(kind: str) -> Callable[[type[T]], type[T]]:
    return _register(POSITION_ENCODINGS, "position_encoding", kind)


def register_block(kind: str) -> Callable[[type[T]], type[T]]:
    return _register(BLOCKS, "block", kind)


def register_embedding(kind: str) -> Callable[[type[T]], type[T]]:
    return _register(EMBEDDINGS, "embedding", kind)


def register_head(kind: str) -> Callable[[type[T]], type[T]]:
    return _register(HEADS, "head", kind)


def build_part(role: str, spec: PartSpec, prefix: str, runtime: Runtime, **extra: Any) -> Any:
    """Instantiate ``spec`` from the registry of ``role`` (``"mixer"``, ``"feed_forward"``,
    ``"norm"``, ``"position_encoding"``, ``"block"``, ``"embedding"`` or ``"head"``)."""
    table = _TABLES[role]
    try:
        cls = table[spec.kind]
    except KeyError:
        raise KeyError(f"unknown {role} kind {spec.kind!r}; registered: {sorted(table)}") from None
    if getattr(cls, "shareable", False) and not extra:
        key = (role, spec.kind, repr(sorted(spec.params.items())))
        if key not in runtime.shared:
            runtime.shared[key] = cls("", runtime, **dict(spec.params))
        return runtime.shared[key]
    return cls(prefix, runtime, **dict(spec.params), **extra)
