"""A model as data: layer descriptions, and the order in which layers run.

An architecture turns its typed configuration into a `ModelSpec`.  Each
`LayerSpec` names its block arrangement and, inside it, the kind of norm, mixer
and feed-forward with their sizes, so one model can mix kinds layer by layer.
`order` is the list of layer calls of a forward pass: it may name a layer twice
(its weights are used again, each call with a cache of its own), and a call may
read the keys and values another call wrote instead of writing its own.
"""

from __future__ import annotations

import dataclasses
from typing import Any, Callable


@dataclasses.dataclass(frozen=True)
class LayerSpec:
    prefix: str  # checkpoint prefix of the layer, e.g. "model.layers.3."
    block: dict[str, Any]  # {"kind": arrangement, "norm": {...}, "mixer": {...}, "feed_forward": {...}, "names": {...}}


@dataclasses.dataclass(frozen=True)
class LayerCall:
    layer: int  # index into ModelSpec.layers
    reads_cache_of: int | None = None  # index of an earlier call in `order`, or None for its own cache


@dataclasses.dataclass(frozen=True)
class ModelSpec:
    vocab_size: int
    hidden_size: int
    embedding_name: str
    layers: list[LayerSpec]
    order: list[LayerCall]
    final_norm: dict[str, Any]
    final_norm_prefix: str
    head_name: str
    tie_word_embeddings: bool
    max_position_embeddings: int | None = None
    # How the residual stream starts and how it ends, by kind like every other part
    # ({"kind": ..., ...}).  None: the plain table lookup under `embedding_name`, and the
    # plain product with the matrix under `head_name` (the table itself when tied).
    embedding: dict[str, Any] | None = None
    head: dict[str, Any] | None = None

    def embedding_description(self) -> dict[str, Any]:
        if self.embedding is not None:
            return self.embedding
        return {"kind": "token_embedding", "vocab_size": self.vocab_size, "hidden_size": self.hidden_size,
                "name": self.embedding_name}

    def head_description(self) -> dict[str, Any]:
        if self.head is not None:
            return self.head
        return {"kind": "linear_head", "vocab_size": self.vocab_size, "hidden_size": self.hidden_size,
                "name": self.head_name, "tied": self.tie_word_embeddings}

    def __post_init__(self) -> None:
        for i, call in enumerate(self.order):
            if not 0 <= call.layer < len(self.layers):
                raise ValueError(f"call {i} names layer {call.layer}, but there are {len(self.layers)} layers")
            if call.reads_cache_of is not None:
                if not 0 <= call.reads_cache_of < i:
                    raise ValueError(f"call {i} reads the cache of call {call.reads_cache_of}, which is not earlier")
                if self.order[call.reads_cache_of].reads_cache_of is not None:
                    raise ValueError(f"call {i} reads the cache of call {call.reads_cache_of}, which owns none")


@dataclasses.dataclass(frozen=True)
class Architecture:
    """What the registry holds for one `architectures[0]` name."""

    name: str
    parse_config: Callable[[dict[str, Any]], Any]  # raw config.json keys -> typed config
    build_spec: Callable[[Any], ModelSpec]  # typed config -> ModelSpec
