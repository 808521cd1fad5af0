"""Arrangement of a layer's parts around the residual stream.

`PreNormBlock` is the reference's `TransformerBlock` with `defer_add=True`
(models/blocks/transformer_block.py:95-120): norm, mixer, add+norm,
feed-forward; the block's own last add is left to the next norm
(`run_decoder_layers`, :142-153).
"""

from __future__ import annotations

import torch

from mini_infer_amd.parts.base import (
    Block,
    FeedForward,
    LayerCache,
    Mixer,
    Norm,
    ParamSpec,
    StepContext,
    TensorGetter,
)
from mini_infer_amd.registry import FEED_FORWARDS, MIXERS, NORMS, register_block


class PreNormBlock(Block):
    def __init__(
        self,
        mixer_norm: Norm,
        mixer: Mixer,
        ffn_norm: Norm,
        feed_forward: FeedForward,
        names: dict[str, str],
        dtype: torch.dtype,
        device,
    ) -> None:
        super().__init__(dtype, device)
        self.mixer_norm = mixer_norm
        self.mixer = mixer
        self.ffn_norm = ffn_norm
        self.feed_forward = feed_forward
        self.names = names  # part -> its prefix inside the layer, e.g. "self_attn."
        # Where all three say they can, the mixer leaves its last product to the norm that
        # follows, and that norm leaves the rows' factors to the feed-forward's first product:
        # for few rows one launch between two weight-streaming products is saved.
        if mixer.can_defer_output and ffn_norm.takes_pending_products and feed_forward.takes_scaled_rows:
            mixer.emit_pending_output = True
            ffn_norm.emit_scaled_rows = True
            ffn_norm.scaled_rows_consumer = feed_forward
        # The same between the block before this one and this block's mixer: its first norm may
        # be handed a product not made yet (if the model arranges that, `enable_pending_output`
        # of the block before), and leaves the rows' factors to the mixer's first product.
        if mixer_norm.takes_pending_products and mixer.takes_scaled_rows:
            mixer_norm.emit_scaled_rows = True
            mixer_norm.scaled_rows_consumer = mixer

    @property
    def graph_safe(self) -> bool:  # type: ignore[override]
        return all(part.graph_safe for _, part in self._children())

    @property
    def takes_partial_sums(self) -> bool:  # type: ignore[override]
        return self.mixer_norm.takes_partial_sums and self.ffn_norm.takes_partial_sums

    def enable_partial_sums(self) -> None:
        self.mixer.emit_partial_sums = True
        self.feed_forward.emit_partial_sums = True

    @property
    def takes_pending_products(self) -> bool:  # type: ignore[override]
        return self.mixer_norm.takes_pending_products

    def enable_pending_output(self) -> None:
        if self.feed_forward.can_defer_output:
            self.feed_forward.emit_pending_output = True

    def _children(self):
        return (
            (self.names["mixer_norm"], self.mixer_norm),
            (self.names["mixer"], self.mixer),
            (self.names["ffn_norm"], self.ffn_norm),
            (self.names["feed_forward"], self.feed_forward),
        )

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        specs: dict[str, ParamSpec] = {}
        for sub, part in self._children():
            specs.update(part.param_specs(prefix + sub))
        return specs

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        for sub, part in self._children():
            part.load_params(prefix + sub, get)

    def forward(
        self,
        delta: torch.Tensor | None,
        residual: torch.Tensor,
        ctx: StepContext,
        cache: LayerCache,
        writes_cache: bool = True,
    ) -> torch.Tensor:
        h = self.mixer_norm.forward(delta, residual)
        mixed = self.mixer.forward(h, ctx, cache, writes_cache)
        h = self.ffn_norm.forward(mixed, residual)
        return self.feed_forward.forward(h, ctx)


@register_block("pre_norm")
def build_pre_norm_block(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> PreNormBlock:
    """`desc` holds `norm`, `mixer` and `feed_forward` descriptions (each with a `kind`)
    and `names`, the prefix of each part inside the layer."""
    shared = {} if shared is None else shared
    norm_desc, mixer_desc, ffn_desc = desc["norm"], desc["mixer"], desc["feed_forward"]
    return PreNormBlock(
        NORMS.lookup(norm_desc["kind"])(norm_desc, dtype, device, shared),
        MIXERS.lookup(mixer_desc["kind"])(mixer_desc, dtype, device, shared),
        NORMS.lookup(norm_desc["kind"])(norm_desc, dtype, device, shared),
        FEED_FORWARDS.lookup(ffn_desc["kind"])(ffn_desc, dtype, device, shared),
        dict(desc["names"]),
        dtype,
        device,
    )
