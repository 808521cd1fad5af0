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
    """What `DecoderModel` builds: embedding part -> layer calls in `order` -> final norm -> head part.

    How the residual stream starts and how it ends is given by kind like every other part:
    `embedding` and `head` are descriptions ({"kind": ..., ...}).  The plain case has a short
    form: with `embedding=None` the table lookup under the checkpoint name `embedding_name`,
    with `head=None` the product with the matrix under `head_name` (or, with
    `tie_word_embeddings`, with the embedding's table).  A spec that gives descriptions of its
    own needs none of the three short-form fields.
    """

    vocab_size: int
    hidden_size: int
    layers: list[LayerSpec]
    order: list[LayerCall]
    final_norm: dict[str, Any]
    final_norm_prefix: str
    embedding_name: str | None = None
    head_name: str | None = None
    tie_word_embeddings: bool = False
    max_position_embeddings: int | None = None
    embedding: dict[str, Any] | None = None
    head: dict[str, Any] | None = None

    def embedding_description(self) -> dict[str, Any]:
        if self.embedding is not None:
            return self.embedding
        if self.embedding_name is None:
            raise ValueError("a ModelSpec needs `embedding` (a part description) or `embedding_name` (the table's checkpoint name)")
        return {"kind": "token_embedding", "vocab_size": self.vocab_size, "hidden_size": self.hidden_size,
                "name": self.embedding_name}

    def head_description(self) -> dict[str, Any]:
        if self.head is not None:
            return self.head
        if self.head_name is None and not self.tie_word_embeddings:
            raise ValueError("a ModelSpec needs `head` (a part description), `head_name` or `tie_word_embeddings`")
        return {"kind": "linear_head", "vocab_size": self.vocab_size, "hidden_size": self.hidden_size,
                "name": self.head_name or "", "tied": self.tie_word_embeddings}

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
    """What the registry holds for one `architectures[0]` name.

    `build_spec` is the usual way: a decoder-only stack as data, built by `DecoderModel`.  An
    architecture of another overall shape (an encoder beside the decoder, two heads) gives
    `build_model(config, dtype, device)` instead and returns any object with the model
    contract, which is all the loader, the random-weights mode, the cache manager and the
    runner ask of a model:

      dtype, device, vocab_size       attributes; `max_position_embeddings` (optional, may be None)
      graph_safe                      whether a step of single tokens may be recorded and replayed
      param_specs()                   {checkpoint name: ParamSpec} of every tensor it loads
      optional_names()                names a checkpoint may hold without the model needing them
      load_params(get)                fetch the tensors by name (`get(name)` -> tensor on the device)
      cache_needs(page_size)          one `CacheNeeds | None` per cache the forward pass uses
      forward(ctx, caches)            logits [len(ctx.logit_rows), vocab] float32 for a `StepContext`
                                      and the `LayerCache`s, in the order of `cache_needs`
    """

    name: str
    parse_config: Callable[[dict[str, Any]], Any]  # raw config.json keys -> typed config
    build_spec: Callable[[Any], ModelSpec] | None = None  # typed config -> ModelSpec
    build_model: Callable[[Any, Any, Any], Any] | None = None  # (typed config, dtype, device) -> model

    def __post_init__(self) -> None:
        if (self.build_spec is None) == (self.build_model is None):
            raise ValueError(f"architecture {self.name!r} gives `build_spec` or `build_model`, one of the two")

    def make_model(self, config: Any, dtype: Any, device: Any) -> Any:
        """The model of a parsed configuration, without weights."""
        if self.build_model is not None:
            return self.build_model(config, dtype, device)
        from mini_infer_amd.models.decoder import DecoderModel

        return DecoderModel(self.build_spec(config), dtype, device)
