"""The parts a model is assembled from; importing this package registers the built-in kinds."""

from turboserve_amd.parts import attention, block, ends, mlp, norm, rope  # noqa: F401  (registration)
from turboserve_amd.parts.base import (  # noqa: F401
    Block,
    CacheNeed,
    Embedding,
    FeedForward,
    FixedState,
    FixedStateView,
    Head,
    Mixer,
    Norm,
    PagedKV,
    PagedKVView,
    Part,
    PartSpec,
    PositionEncoding,
    ResidualStream,
    Runtime,
    TensorSpec,
)
from turboserve_amd.parts.registry import (  # noqa: F401
    build_part,
    register_block,
    register_embedding,
    register_feed_forward,
    register_head,
    register_mixer,
    register_norm,
    register_position_encoding,
)
