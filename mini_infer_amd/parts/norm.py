"""RMSNorm with the residual add folded in.

Formula: models/blocks/rmsnorm.py:81-93 of the reference; the add-then-norm
pairing is its `_add_and_norm` (:63-79) and kernel (rms_norm_kernel.py:109-144).
Here the residual stream is float32 in both compute dtypes, so the sum is
exact to float32 and the statistics see the unrounded sum.
"""

from __future__ import annotations

import torch

from mini_infer_amd import ops
from mini_infer_amd.parts.base import Norm, ParamSpec, TensorGetter
from mini_infer_amd.registry import register_norm


class RMSNorm(Norm):
    graph_safe = True
    takes_partial_sums = True
    takes_pending_products = True

    def __init__(self, hidden_size: int, eps: float, dtype: torch.dtype, device) -> None:
        super().__init__(dtype, device)
        self.hidden_size = hidden_size
        self.eps = float(eps)
        self.weight: torch.Tensor | None = None

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        return {prefix + "weight": ParamSpec((self.hidden_size,), init="norm_weight")}

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        self.weight = get(prefix + "weight").contiguous()

    def forward(
        self,
        delta: "torch.Tensor | ops.PartialSums | ops.PendingProduct | None",
        residual: torch.Tensor,
        rows: torch.Tensor | None = None,
    ) -> "torch.Tensor | ops.ScaledRows":
        assert self.weight is not None, "RMSNorm used before its weight was loaded"
        if isinstance(delta, ops.PendingProduct):
            # few rows: the product, the add and the norm but for the rows' factors are one
            # kernel, if the part that follows has a kernel that applies the factors in this step
            consumer = self.scaled_rows_consumer
            if (
                self.emit_scaled_rows
                and rows is None
                and consumer is not None
                and consumer.wants_scaled_rows(residual.shape[0])
                and ops.linear_add_norm_takes(delta, residual, self.weight)
            ):
                return ops.linear_add_norm(delta, residual, self.weight, self.eps)
            delta = delta.finish()
        return ops.add_rmsnorm(delta, residual, self.weight, self.eps, rows)


@register_norm("rms_norm")
def build_rms_norm(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> RMSNorm:
    return RMSNorm(int(desc["hidden_size"]), float(desc["eps"]), dtype, device)
