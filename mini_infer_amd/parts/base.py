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
    """What a mixer keeps per token in pages: per key/value head one key row of `head_dim`
    values and one value row of `v_head_dim` values (None: as wide as the keys; 0: no value
    stream at all, the mixer keeps a single stream and gets no value pages).

    `window=None` keeps every token; with a window, pages that no future query can see
    are given back.  `v_transposed` is the layout of a value page, chosen by the mixer
    for the kernel that will read it: `[slot][dim]` (False) or `[dim][slot]` (True).
    Layer calls whose needs are equal share one page group.
    """

    num_kv_heads: int
    head_dim: int
    window: int | None = None
    v_head_dim: int | None = None
    v_transposed: bool = False

    @property
    def value_dim(self) -> int:
        return self.head_dim if self.v_head_dim is None else self.v_head_dim


@dataclasses.dataclass(frozen=True)
class StateNeeds:
    """A tensor of fixed size per request, zero when the request is admitted."""

    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclasses.dataclass(frozen=True)
class CacheNeeds:
    """What one call of a mixer keeps per request: pages, state of fixed size, both or neither.

    `state` is one `StateNeeds` (the mixer then finds one tensor under `LayerCache.state`) or a
    mapping of names to `StateNeeds` (a dict of tensors under the same names): a mixer with a
    short convolution tail in the compute dtype beside a float32 recurrent state asks for
    `{"tail": StateNeeds((width, 3), dtype), "recurrent": StateNeeds((heads, d, d))}`.
    """

    pages: PagedKVNeeds | None = None
    state: "StateNeeds | dict[str, StateNeeds] | None" = None


@dataclasses.dataclass
class LayerCache:
    """The cache of one layer call: views the cache manager hands to a mixer."""

    group: int | None = None  # which page group's block table and write slots apply
    k_pages: torch.Tensor | None = None  # [num_pages, kv_heads, page_size, head_dim]
    # [num_pages, kv_heads, page_size, value dim], or [num_pages, kv_heads, value dim, page_size]
    # if transposed; None for a mixer that asked for no value stream
    v_pages: torch.Tensor | None = None
    v_transposed: bool = False
    # [max_requests + 1, *state shape], one row per state slot (the last row is nobody's: slot -1);
    # a dict of such tensors by name if the mixer asked for several
    state: "torch.Tensor | dict[str, torch.Tensor] | None" = None


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
    # Host copies, for parts that loop over requests on the host or shape a launch by the
    # requests' lengths.  None in a step that is being recorded to be replayed with other
    # boundaries (only models whose parts are all `graph_safe` are recorded): `num_tokens`,
    # `num_requests`, `max_q_len` and `max_seq_len` are then upper bounds that hold for every
    # replay, some requests may bring no token at all, and everything else about the step is
    # to be read from the device tensors.
    host_cu_seqlens_q: list[int] | None = dataclasses.field(default_factory=list)
    host_seq_lens: list[int] | None = dataclasses.field(default_factory=list)
    host_state_slots: list[int] | None = dataclasses.field(default_factory=list)
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

    `takes_pending_products`: `delta` may also be an `ops.PendingProduct` (a product not made
    yet); and where the block has set `emit_scaled_rows` on the norm, because the part that
    consumes its output says `takes_scaled_rows`, the norm may return `ops.ScaledRows`
    (its output but for the rows' factors) instead of a tensor.  Both are a block's own
    arrangement between its parts: a norm that knows neither is fine.
    """

    takes_partial_sums = False
    takes_pending_products = False
    emit_scaled_rows = False
    # the part that consumes this norm's output, set by the block together with
    # `emit_scaled_rows`; the norm asks its `wants_scaled_rows(rows)` step by step
    scaled_rows_consumer = None

    def forward(
        self,
        delta: torch.Tensor | None,
        residual: torch.Tensor,
        rows: torch.Tensor | None = None,
    ) -> torch.Tensor:
        raise NotImplementedError


@dataclasses.dataclass
class RotaryTables:
    """Rotation of the first `rotary_dim` dims of every query and key head by the angle of
    its token: `cos`, `sin` are float32 [T, rotary_dim/2] for the step's tokens;
    `interleaved` pairs dim 2j with 2j+1, otherwise j with j + rotary_dim/2."""

    cos: torch.Tensor
    sin: torch.Tensor
    rotary_dim: int
    interleaved: bool = False


class PositionEncoding(Part):
    """How a mixer learns where its tokens are.  An attention mixer asks two things of it,
    each of which may answer None ("not my way of encoding positions"):

    `rotary(ctx)`: tables to rotate queries and keys with before the scores are taken.

    `score_slopes(num_heads)`: a float32 tensor [num_heads] on the device; the score of
    query head h at position p for the key at position j gets `slopes[h] * (j - p)` added
    before the softmax (a penalty linear in the distance for positive slopes).

    An encoding that acts elsewhere (learned positions added to the embedding, say) is an
    `Embedding` part's business and answers None to both.
    """

    def rotary(self, ctx: "StepContext") -> RotaryTables | None:
        return None

    def rotary_layout(self) -> tuple[int, bool] | None:
        """`(rotary_dim, interleaved)` of the tables `rotary` will return, if that is the same
        for every step, else None.  Lets a mixer say before a step which of its kernels the
        step will take; an encoding that does not answer costs nothing but that foresight."""
        return None

    def score_slopes(self, num_heads: int) -> torch.Tensor | None:
        return None


class Mixer(Part):
    """Mixes tokens of one request: attention here, anything with a cache or a state.

    `emit_partial_sums` is set by the model, never by the part: when true, `forward` may
    return an `ops.PartialSums` instead of a tensor (parts that ignore it are fine).
    `emit_pending_output` is set by the block where the norm that follows says
    `takes_pending_products` and the mixer `can_defer_output`: `forward` may then return an
    `ops.PendingProduct` (its last product, not made yet) instead of a tensor.
    `takes_scaled_rows`: `x` may be an `ops.ScaledRows` (a norm's output but for the rows'
    factors); the block then lets the norm before the mixer emit them, and the norm asks
    `wants_scaled_rows(rows)` before it does so in a step of `rows` rows."""

    emit_partial_sums = False
    can_defer_output = False
    emit_pending_output = False
    takes_scaled_rows = False

    def wants_scaled_rows(self, rows: int) -> bool:
        """Whether, in a step of `rows` rows, the part has a kernel that applies the rows'
        factors itself.  A part that answers False gets a finished tensor."""
        return self.takes_scaled_rows

    def cache_needs(self, page_size: int) -> CacheNeeds:
        """What the cache manager must keep for one call of this mixer, given its page size
        (a mixer may choose its page layout by it)."""
        return CacheNeeds()

    def forward(
        self, x: torch.Tensor, ctx: StepContext, cache: LayerCache, writes_cache: bool = True
    ) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    """Acts on each token alone: dense or routed experts.  `emit_partial_sums`: as for `Mixer`.
    `takes_scaled_rows`: `x` may be an `ops.ScaledRows` (a norm's output but for the rows'
    factors).  `can_defer_output`, `emit_pending_output`: as for `Mixer`; here it is the
    model that sets the latter (`Block.enable_pending_output`), since the norm that follows
    belongs to whatever comes next in the model's order."""

    emit_partial_sums = False
    takes_scaled_rows = False
    can_defer_output = False
    emit_pending_output = False

    def wants_scaled_rows(self, rows: int) -> bool:
        """As `Mixer.wants_scaled_rows`."""
        return self.takes_scaled_rows

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        raise NotImplementedError


class Embedding(Part):
    """Starts the float32 residual stream of a step: `forward(ctx)` -> [T, hidden] float32
    from `ctx.token_ids` (and, if it wishes, `ctx.positions`)."""

    def forward(self, ctx: StepContext) -> torch.Tensor:
        raise NotImplementedError


class Head(Part):
    """Ends a step: `forward(h, ctx)` takes the normalized rows [rows, hidden] in the compute
    dtype and returns logits [rows, vocab] in float32.  `optional_names(prefix)` lists
    tensors a checkpoint may hold without the head needing them."""

    def optional_names(self, prefix: str) -> set[str]:
        return set()

    def forward(self, h: torch.Tensor, ctx: StepContext) -> torch.Tensor:
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

    # Whether the block's `delta` may be an `ops.PendingProduct` (the previous block's last
    # product, not made yet).  Where everything that follows a block in the model's order (the
    # blocks after it, the final norm after the last) says so, the model calls the block's
    # `enable_pending_output()`, which lets its last part hand its last product on unmade.
    takes_pending_products = False

    def enable_pending_output(self) -> None:
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
