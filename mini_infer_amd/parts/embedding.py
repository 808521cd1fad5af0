"""Token embedding and output head.

Embedding: a row lookup that starts the float32 residual stream
(models/llama/llama.py:159 of the reference).  Head: `logits = h @ W.T` on the
requested rows only (llama.py:169-171); with tied embeddings the head's matrix is
the embedding table and the checkpoint holds no `lm_head.weight` (llama.py:143-147).

Both are chosen by kind like every other part, so a model whose stream starts or
ends differently (a scaled embedding, learned positions added to it, capped logits)
registers a part of its own and names it in its `ModelSpec`.
"""

from __future__ import annotations

import torch

from mini_infer_amd import ops
from mini_infer_amd.parts.base import Embedding, Head, ParamSpec, StepContext, TensorGetter
from mini_infer_amd.registry import register_embedding, register_head


class TokenEmbedding(Embedding):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, name: str, dtype: torch.dtype, device) -> None:
        super().__init__(dtype, device)
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.name = name
        self.weight: torch.Tensor | None = None

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        return {prefix + self.name: ParamSpec((self.vocab_size, self.hidden_size))}

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        self.weight = get(prefix + self.name).contiguous()

    def forward(self, ctx: StepContext) -> torch.Tensor:
        assert self.weight is not None, "embedding used before its table was loaded"
        return ops.embed_gather(self.weight, ctx.token_ids)


class OutputHead(Head):
    graph_safe = True

    def __init__(
        self,
        hidden_size: int,
        vocab_size: int,
        name: str,
        dtype: torch.dtype,
        device,
        *,
        tied_to: TokenEmbedding | None = None,
    ) -> None:
        super().__init__(dtype, device)
        self.hidden_size = hidden_size
        self.vocab_size = vocab_size
        self.name = name
        self.tied_to = tied_to
        self._weight: torch.Tensor | None = None

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        if self.tied_to is not None:
            return {}
        return {prefix + self.name: ParamSpec((self.vocab_size, self.hidden_size))}

    def optional_names(self, prefix: str) -> set[str]:
        """Names a checkpoint may hold without the model needing them."""
        return {prefix + self.name} if self.tied_to is not None else set()

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        if self.tied_to is None:
            self._weight = get(prefix + self.name).contiguous()

    @property
    def weight(self) -> torch.Tensor:
        w = self.tied_to.weight if self.tied_to is not None else self._weight
        assert w is not None, "output head used before its matrix was loaded"
        return w

    def forward(self, h: torch.Tensor, ctx: StepContext | None = None) -> torch.Tensor:
        """Logits [rows, vocab] in float32."""
        return ops.linear_f32_out(h, self.weight)


@register_embedding("token_embedding")
def build_token_embedding(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> TokenEmbedding:
    return TokenEmbedding(int(desc["vocab_size"]), int(desc["hidden_size"]), str(desc["name"]), dtype, device)


@register_head("linear_head")
def build_linear_head(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> OutputHead:
    """`desc["tied"]`: the head's matrix is the table of the model's embedding part (which the
    model leaves under `shared["embedding"]` before it builds the head)."""
    tied_to = None
    if desc.get("tied", False):
        tied_to = (shared or {}).get("embedding")
        if tied_to is None or not hasattr(tied_to, "weight"):
            raise ValueError("a tied output head needs the model's embedding part to hold a `weight` table")
    return OutputHead(
        int(desc["hidden_size"]), int(desc["vocab_size"]), str(desc["name"]), dtype, device, tied_to=tied_to
    )
