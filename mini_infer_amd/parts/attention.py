"""Grouped-query attention over the paged cache.

Order of operations as in the reference's `GroupedQueryAttention.forward`
(models/blocks/gqa.py:107-154): one merged q|k|v projection, rotary encoding of
q and k fused with the write of k and v into cache pages
(rope_write_kernel.py:75-152), causal attention over the pages with scale
1/sqrt(head_dim) (cache/packed_attention.py:126-127, :296-338), output
projection.  A window, if given, limits each query to the last `window` keys.
"""

from __future__ import annotations

import math

import torch

from mini_infer_amd import ops
from mini_infer_amd.parts.base import (
    CacheNeeds,
    LayerCache,
    Mixer,
    PagedKVNeeds,
    ParamSpec,
    PositionEncoding,
    StepContext,
    TensorGetter,
)
from mini_infer_amd.parts.linear import Linear
from mini_infer_amd.registry import POSITION_ENCODINGS, register_mixer


class GQAttention(Mixer):
    graph_safe = True
    can_defer_output = True
    takes_scaled_rows = True

    def __init__(
        self,
        hidden_size: int,
        num_heads: int,
        num_kv_heads: int,
        head_dim: int,
        position: PositionEncoding | None,
        dtype: torch.dtype,
        device,
        *,
        window: int | None = None,
        scale: float | None = None,
    ) -> None:
        super().__init__(dtype, device)
        if num_heads % num_kv_heads != 0:
            raise ValueError(f"num_heads={num_heads} is not a multiple of num_kv_heads={num_kv_heads}")
        if window is not None and window <= 0:
            raise ValueError(f"window must be positive, got {window}")
        if head_dim <= 0 or head_dim % ops.ATTENTION_HEAD_DIM_STEP != 0 or head_dim > ops.ATTENTION_MAX_HEAD_DIM:
            raise ValueError(
                f"head_dim={head_dim}: the attention kernels take even head sizes "
                f"up to {ops.ATTENTION_MAX_HEAD_DIM}"
            )
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.position = position
        self.window = window
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        # per-head slopes of a score bias linear in the distance, if the encoding has one
        self.slopes = position.score_slopes(num_heads) if position is not None else None
        if self.slopes is not None and (
            self.slopes.dtype != torch.float32 or tuple(self.slopes.shape) != (num_heads,)
        ):
            raise ValueError(f"score slopes must be float32 [{num_heads}], got {self.slopes.dtype} {tuple(self.slopes.shape)}")
        q_width, kv_width = num_heads * head_dim, num_kv_heads * head_dim
        self.qkv = Linear(hidden_size, [q_width, kv_width, kv_width], ["q_proj", "k_proj", "v_proj"], dtype, device)
        self.out = Linear(q_width, hidden_size, "o_proj", dtype, device)

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        return {**self.qkv.param_specs(prefix), **self.out.param_specs(prefix)}

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        self.qkv.load_params(prefix, get)
        self.out.load_params(prefix, get)

    def wants_scaled_rows(self, rows: int) -> bool:
        """Only where projection, rotation and cache write will run as the one kernel that
        applies the rows' factors: few bfloat16 rows, whole heads rotated in half pairing."""
        layout = self.position.rotary_layout() if self.position is not None else None
        return (
            self.dtype == torch.bfloat16
            and layout == (self.head_dim, False)
            and self.head_dim % 32 == 0
            and ops.scaled_rows_product_takes(rows, self.qkv.weight, self.hidden_size)
        )

    def cache_needs(self, page_size: int) -> CacheNeeds:
        # values lie transposed inside a page where the matrix-core kernel will read them
        # (that kernel knows no score bias: such layers keep the plain layout and kernel)
        transposed = self.slopes is None and ops.mfma_attention_supported(self.dtype, self.head_dim, page_size)
        return CacheNeeds(
            pages=PagedKVNeeds(self.num_kv_heads, self.head_dim, self.window, v_transposed=transposed)
        )

    def forward(
        self, x: torch.Tensor, ctx: StepContext, cache: LayerCache, writes_cache: bool = True
    ) -> torch.Tensor:
        assert cache.group is not None and cache.k_pages is not None and cache.v_pages is not None
        q_width = self.num_heads * self.head_dim
        assert self.qkv.weight is not None
        rotary = self.position.rotary(ctx) if self.position is not None else None
        if isinstance(x, ops.ScaledRows) and not (
            rotary is not None
            and ops.qkv_rope_write_takes(x, self.qkv.weight, self.head_dim, rotary.rotary_dim, rotary.interleaved)
        ):
            x = x.finish()  # rows but for their norm factors, and no kernel here that applies them
        if rotary is not None and ops.qkv_rope_write_takes(
            x, self.qkv.weight, self.head_dim, rotary.rotary_dim, rotary.interleaved
        ):
            # few rows (decode): projection, rotation and cache write are one kernel
            kv_heads = self.num_kv_heads if writes_cache else 0
            queries = ops.qkv_rope_write(
                x, self.qkv.weight if writes_cache else self.qkv.weight[:q_width], rotary.cos, rotary.sin,
                ctx.slot_mapping[cache.group] if writes_cache else None, cache.k_pages, cache.v_pages,
                q_heads=self.num_heads, kv_heads=kv_heads, head_dim=self.head_dim,
                v_transposed=cache.v_transposed,
            )
            return self._project(self._attend(queries, ctx, cache))
        if writes_cache:
            qkv = self.qkv.forward(x)
            kv_heads, slots = self.num_kv_heads, ctx.slot_mapping[cache.group]
        else:
            # reads another call's keys and values: only q is projected
            qkv = ops.linear(x, self.qkv.weight[:q_width])
            kv_heads, slots = 0, None
        if rotary is not None:
            cos, sin, rotary_dim, interleaved = rotary.cos, rotary.sin, rotary.rotary_dim, rotary.interleaved
        else:
            cos = sin = torch.empty((ctx.num_tokens, 0), dtype=torch.float32, device=x.device)
            rotary_dim, interleaved = 0, False
        ops.rope_kv_write(
            qkv, cos, sin, slots, cache.k_pages, cache.v_pages,
            q_heads=self.num_heads, kv_heads=kv_heads, head_dim=self.head_dim,
            rotary_dim=rotary_dim, interleaved=interleaved, v_transposed=cache.v_transposed,
        )
        return self._project(self._attend(qkv, ctx, cache))

    def _project(self, attended):
        """The output projection of what `_attend` returned; for few rows, where the block
        asked for it, not made here but handed on to the norm that follows."""
        assert self.out.weight is not None
        if self.emit_pending_output and self.dtype == torch.bfloat16:
            rows = attended.tokens if isinstance(attended, ops.AttentionPieces) else attended.shape[0]
            q_width = self.num_heads * self.head_dim
            if ops.pending_product_pays(rows, self.hidden_size, q_width, self.emit_partial_sums):
                return ops.PendingProduct(attended, self.out.weight)
        if isinstance(attended, ops.AttentionPieces):
            return ops.linear_from_attention(attended, self.out.weight)
        return self.out.forward(attended, partial_ok=self.emit_partial_sums)

    def _attend(self, queries: torch.Tensor, ctx: StepContext, cache: LayerCache):
        """Attention of the rotated queries (the first columns of `queries`) over the cache pages.
        At the smallest batches the key ranges may come back uncombined, for the output
        projection to combine on its way (one launch less a layer)."""
        few = queries.dtype == torch.bfloat16 and ops.attention_pieces_pay(ctx.num_tokens, self.num_heads, self.head_dim)
        return ops.paged_attention(
            queries, cache.k_pages, cache.v_pages, ctx.block_tables[cache.group], ctx.token_request,
            ctx.positions, ctx.cu_seqlens_q, ctx.host_cu_seqlens_q, q_heads=self.num_heads,
            kv_heads=self.num_kv_heads, head_dim=self.head_dim, scale=self.scale, window=self.window,
            max_seq_len=ctx.max_seq_len, v_transposed=cache.v_transposed, combine=not few, slopes=self.slopes,
        )


@register_mixer("gqa_attention")
def build_gqa_attention(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> GQAttention:
    position = None
    pos_desc = desc.get("position")
    if pos_desc is not None:
        key = ("position", repr(sorted(pos_desc.items(), key=lambda kv: kv[0])))
        if shared is not None and key in shared:
            position = shared[key]
        else:
            position = POSITION_ENCODINGS.lookup(pos_desc["kind"])(pos_desc, dtype, device, shared)
            if shared is not None:
                shared[key] = position
    return GQAttention(
        int(desc["hidden_size"]),
        int(desc["num_heads"]),
        int(desc["num_kv_heads"]),
        int(desc["head_dim"]),
        position,
        dtype,
        device,
        window=desc.get("window"),
        scale=desc.get("scale"),
    )
