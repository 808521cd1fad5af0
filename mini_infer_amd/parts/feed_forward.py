"""Dense gated feed-forward: `down(silu(gate(x)) * up(x))`, no biases.

Formula: models/blocks/swiglu.py:44-46 and activations.py:36-45 of the
reference.  Gate and up are two tensors in the checkpoint; they are stacked at
load so one product yields [gate | up], and the activation reads both halves
(the reference runs two products and one fused SiLU*mul kernel); for few rows
the product and the activation are one kernel.
"""

from __future__ import annotations

import torch

from mini_infer_amd import ops
from mini_infer_amd.parts.base import FeedForward, ParamSpec, StepContext, TensorGetter
from mini_infer_amd.parts.linear import Linear
from mini_infer_amd.registry import register_feed_forward


class SwiGLU(FeedForward):
    graph_safe = True
    takes_scaled_rows = True
    can_defer_output = True

    def __init__(self, hidden_size: int, intermediate_size: int, dtype: torch.dtype, device) -> None:
        super().__init__(dtype, device)
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.gate_up = Linear(
            hidden_size, [intermediate_size, intermediate_size], ["gate_proj", "up_proj"], dtype, device
        )
        self.down = Linear(intermediate_size, hidden_size, "down_proj", dtype, device)

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        return {**self.gate_up.param_specs(prefix), **self.down.param_specs(prefix)}

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        self.gate_up.load_params(prefix, get)
        self.down.load_params(prefix, get)

    def wants_scaled_rows(self, rows: int) -> bool:
        """Where the gated product runs as the weight-streaming kernel that applies the rows' factors."""
        return self.dtype == torch.bfloat16 and ops.scaled_rows_product_takes(rows, self.gate_up.weight, self.hidden_size)

    def forward(self, x: "torch.Tensor | ops.ScaledRows", ctx: StepContext) -> torch.Tensor:
        assert self.gate_up.weight is not None, "SwiGLU used before its weights were loaded"
        assert self.down.weight is not None
        act = ops.linear_swiglu(x, self.gate_up.weight)
        if (
            self.emit_pending_output
            and self.dtype == torch.bfloat16
            and ops.pending_product_pays(act.shape[0], self.hidden_size, self.intermediate_size, self.emit_partial_sums)
        ):
            # few rows: the down product is left to the norm that follows (one kernel makes it,
            # adds it to the residual and begins the norm)
            return ops.PendingProduct(act, self.down.weight)
        return self.down.forward(act, partial_ok=self.emit_partial_sums)


@register_feed_forward("swiglu")
def build_swiglu(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> SwiGLU:
    activation = desc.get("activation", "silu")
    if activation != "silu":
        raise NotImplementedError(f"gated feed-forward activation {activation!r}; only 'silu' is built")
    return SwiGLU(int(desc["hidden_size"]), int(desc["intermediate_size"]), dtype, device)
