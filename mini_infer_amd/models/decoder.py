"""A decoder-only language model assembled from a `ModelSpec`.

Embedding part -> layer calls in `spec.order` -> final norm at the requested rows ->
head part, the reference's `LlamaForCausalLM.forward`
(models/llama/llama.py:149-172) with `run_decoder_layers`
(models/blocks/transformer_block.py:123-153), but driven by data: nothing here
names an architecture.
"""

from __future__ import annotations

import torch

from mini_infer_amd.models.spec import ModelSpec
from mini_infer_amd.parts.base import (
    Block,
    CacheNeeds,
    LayerCache,
    ParamSpec,
    StepContext,
    TensorGetter,
)
from mini_infer_amd.registry import BLOCKS, EMBEDDINGS, HEADS, NORMS


class DecoderModel:
    def __init__(self, spec: ModelSpec, dtype: torch.dtype, device) -> None:
        import mini_infer_amd.parts  # noqa: F401  (registers the built-in part kinds)

        self.spec = spec
        self.dtype = dtype
        self.device = torch.device(device)
        shared: dict = {}
        embedding = spec.embedding_description()
        self.embedding = EMBEDDINGS.lookup(embedding["kind"])(embedding, dtype, device, shared)
        shared["embedding"] = self.embedding  # a tied head finds its table here
        self.blocks: list[Block] = [
            BLOCKS.lookup(layer.block["kind"])(layer.block, dtype, device, shared) for layer in spec.layers
        ]
        self.final_norm = NORMS.lookup(spec.final_norm["kind"])(spec.final_norm, dtype, device, shared)
        head = spec.head_description()
        self.head = HEADS.lookup(head["kind"])(head, dtype, device, shared)
        # a product whose output only ever meets norms that can add up its pieces may leave them apart
        if self.final_norm.takes_partial_sums and all(block.takes_partial_sums for block in self.blocks):
            for block in self.blocks:
                block.enable_partial_sums()
        # a block may hand its last product on unmade where whatever follows it, at every place
        # it has in the order, takes such a product
        followers: dict[int, list] = {}
        for i, call in enumerate(spec.order):
            after = self.blocks[spec.order[i + 1].layer] if i + 1 < len(spec.order) else self.final_norm
            followers.setdefault(call.layer, []).append(after)
        for layer, after in followers.items():
            if all(part.takes_pending_products for part in after):
                self.blocks[layer].enable_pending_output()

    @property
    def vocab_size(self) -> int:
        return self.spec.vocab_size

    @property
    def max_position_embeddings(self) -> int | None:
        """The positions the model's encoding was made for (None: no bound is known)."""
        return self.spec.max_position_embeddings

    @property
    def graph_safe(self) -> bool:
        """Whether a decode step of this model can be recorded as a HIP graph."""
        parts = [self.embedding, self.final_norm, self.head, *self.blocks]
        return all(part.graph_safe for part in parts)

    # -- weights --------------------------------------------------------------

    def param_specs(self) -> dict[str, ParamSpec]:
        specs = dict(self.embedding.param_specs(""))
        for layer, block in zip(self.spec.layers, self.blocks):
            specs.update(block.param_specs(layer.prefix))
        specs.update(self.final_norm.param_specs(self.spec.final_norm_prefix))
        specs.update(self.head.param_specs(""))
        return specs

    def optional_names(self) -> set[str]:
        return self.head.optional_names("")

    def load_params(self, get: TensorGetter) -> None:
        self.embedding.load_params("", get)
        for layer, block in zip(self.spec.layers, self.blocks):
            block.load_params(layer.prefix, get)
        self.final_norm.load_params(self.spec.final_norm_prefix, get)
        self.head.load_params("", get)

    # -- cache ----------------------------------------------------------------

    def cache_needs(self, page_size: int) -> list[CacheNeeds | None]:
        """Per call in `order`: what its own cache must hold, or None if it reads another's."""
        return [
            None if call.reads_cache_of is not None else self.blocks[call.layer].mixer.cache_needs(page_size)
            for call in self.spec.order
        ]

    # -- forward --------------------------------------------------------------

    def forward(self, ctx: StepContext, caches: list[LayerCache]) -> torch.Tensor:
        """Logits [len(ctx.logit_rows), vocab] float32.  `caches[i]` belongs to call i."""
        residual = self.embedding.forward(ctx)
        delta: torch.Tensor | None = None
        for i, call in enumerate(self.spec.order):
            own = call.reads_cache_of is None
            cache = caches[i if own else call.reads_cache_of]
            delta = self.blocks[call.layer].forward(delta, residual, ctx, cache, writes_cache=own)
        if ctx.logit_rows.numel() == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=self.device)
        h = self.final_norm.forward(delta, residual, rows=ctx.logit_rows)
        return self.head.forward(h, ctx)
