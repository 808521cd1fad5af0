"""Parts a layer is put together from.  Importing this package registers the built-in kinds."""

from mini_infer_amd.parts import attention, block, embedding, feed_forward, norm, position  # noqa: F401
from mini_infer_amd.parts.base import (
    Block,
    CacheNeeds,
    Embedding,
    FeedForward,
    Head,
    LayerCache,
    Mixer,
    Norm,
    PagedKVNeeds,
    ParamSpec,
    Part,
    PositionEncoding,
    RotaryTables,
    StateNeeds,
    StepContext,
)

__all__ = [
    "Block",
    "CacheNeeds",
    "Embedding",
    "FeedForward",
    "Head",
    "LayerCache",
    "Mixer",
    "Norm",
    "PagedKVNeeds",
    "ParamSpec",
    "Part",
    "PositionEncoding",
    "RotaryTables",
    "StateNeeds",
    "StepContext",
]
