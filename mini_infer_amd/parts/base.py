"""What every part of a layer has in common, and what a step hands to it.

A part (norm, position encoding, mixer, feed-forward, block arrangement) takes
its sizes and constants as constructor arguments, names the tensors it needs,
and runs on the flattened tokens of one step.  No part knows which model it is
in: the model is a list of layer descriptions that name parts by kind.
"""

from __future__ import annotations

import dataclasses
from typing import Callable

import torch


# ----------------------------------------------------------------------------
# parameters
# ----------------------------------------------------------------------------


@dataclasses.dataclass(frozen=True)
class ParamSpec:
    """One tensor a part reads from the checkpoint.

    `init` chooses the random-weights distribution: "normal" is N(0, std),
    "norm_weight" is 1 + N(0, jitter).  `dtype` is "compute" (the engine's
    dtype), "float32" (stays 32-bit whatever the engine's dtype) or "int32".
    """

    shape: tuple[int, ...]
    init: str = "normal"
    dtype: str = "compute"


TensorGetter = Callable[[str], torch.Tensor]


class Part:
    """Base of all parts.  `dtype` is the compute dtype, float32 or bfloat16.

    `graph_safe` says that `forward` only launches device work that depends on the
    step through device tensors (not through host lists or Python loops over
    requests), so a decode step containing the part can be recorded once as a HIP
    graph and replayed.  Parts are not graph-safe unless they say so.
    """

    graph_safe = False

    def __init__(self, dtype: torch.dtype, device: torch.device | str) -> None:
        self.dtype = dtype
        self.device = torch.device(device)

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        """Full tensor name -> spec for everything this part loads."""
        return {}

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        """Fetch this part's tensors (already on device, already cast) by full name."""


# ----------------------------------------------------------------------------
# cache needs
# ----------------------------------------------------------------------------


@dataclasses.dataclass(frozen=True)
class PagedKVNeeds:
    """Keys and values per token, kept in pages.  `window=None` keeps all of them."""

    num_kv_heads: int
    head_dim: int
    window: int | None = None


@dataclasses.dataclass(frozen=True)
class StateNeeds:
    """A tensor of fixed size per request, zero when the request is admitted."""

    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclasses.dataclass(frozen=True)
class CacheNeeds:
    pages: PagedKVNeeds | None = None
    state: StateNeeds | None = None


@dataclasses.dataclass
class LayerCache:
    """The cache of one layer call: views the cache manager hands to a mixer."""

    group: int | None = None  # which page group's block table and write slots apply
    k_pages: torch.Tensor | None = None  # [num_pages, kv_heads, page_size, head_dim]
    v_pages: torch.Tensor | None = None  # same, or [num_pages, kv_heads, head_dim, page_size] if transposed
    v_transposed: bool = False
    state: torch.Tensor | None = None  # [max_requests, *state shape]


# ----------------------------------------------------------------------------
# the step a part runs in
# ----------------------------------------------------------------------------


@dataclasses.dataclass
class StepContext:
    """Device-side description of one step's flattened batch, shared by all layers.

    T tokens of B requests.  Request b owns tokens cu_seqlens_q[b]..cu_seqlens_q[b+1];
    token t sits at absolute position positions[t] of request token_request[t];
    after the step request b holds seq_lens[b] tokens.  Per page group g,
    slot_mapping[g][t] = page * page_size + offset is where token t's keys and
    values go, and block_tables[g][b] lists request b's pages (entries a window
    has passed are -1).
    """

    num_tokens: int
    num_requests: int
    page_size: int
    token_ids: torch.Tensor
    positions: torch.Tensor
    token_request: torch.Tensor
    cu_seqlens_q: torch.Tensor
    seq_lens: torch.Tensor
    state_slots: torch.Tensor
    logit_rows: torch.Tensor
    slot_mapping: list[torch.Tensor]
    block_tables: list[torch.Tensor]
    max_q_len: int
    max_seq_len: int
    # host copies, for parts that loop over requests on the host
    host_cu_seqlens_q: list[int] = dataclasses.field(default_factory=list)
    host_seq_lens: list[int] = dataclasses.field(default_factory=list)
    host_state_slots: list[int] = dataclasses.field(default_factory=list)
    # per-step results shared between layers (rotation tables and the like), by key
    shared: dict = dataclasses.field(default_factory=dict)


# ----------------------------------------------------------------------------
# interfaces
# ----------------------------------------------------------------------------


class Norm(Part):
    """`forward(delta, residual, rows)`.

    Adds `delta` (or nothing) into the float32 residual stream in place and
    returns the normalized sum in the compute dtype.  With `rows`, only those
    rows are normalized and returned, and the residual is left as it was.

    `takes_partial_sums`: `delta` may also be an `ops.PartialSums` (a product whose sums
    over ranges of K are still apart); a model lets its mixers and feed-forwards emit
    those only if every one of its norms says it takes them.
    """

    takes_partial_sums = False

    def forward(
        self,
        delta: torch.Tensor | None,
        residual: torch.Tensor,
        rows: torch.Tensor | None = None,
    ) -> torch.Tensor:
        raise NotImplementedError


class PositionEncoding(Part):
    """Describes how a mixer encodes positions; rotary kinds expose `inv_freq`."""


class Mixer(Part):
    """Mixes tokens of one request: attention here, anything with a cache or a state.

    `emit_partial_sums` is set by the model, never by the part: when true, `forward` may
    return an `ops.PartialSums` instead of a tensor (parts that ignore it are fine)."""

    emit_partial_sums = False

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds()

    def forward(
        self, x: torch.Tensor, ctx: StepContext, cache: LayerCache, writes_cache: bool = True
    ) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    """Acts on each token alone: dense or routed experts.  `emit_partial_sums`: as for `Mixer`."""

    emit_partial_sums = False

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    """An arrangement of norms, a mixer and a feed-forward around the residual stream.

    `forward(delta, residual, ...)` takes the previous block's output still to
    be added (`delta`, None for the first block) and the float32 residual, and
    returns its own pending output; the add happens in the next norm.
    """

    mixer: Mixer

    # Whether every norm of the block takes `ops.PartialSums` as its delta; only if all
    # blocks of a model and its final norm do, the model calls `enable_partial_sums()`,
    # which lets the block's mixer and feed-forward emit them.
    takes_partial_sums = False

    def enable_partial_sums(self) -> None:
        pass

    def forward(
        self,
        delta: torch.Tensor | None,
        residual: torch.Tensor,
        ctx: StepContext,
        cache: LayerCache,
        writes_cache: bool = True,
    ) -> torch.Tensor:
        raise NotImplementedError
