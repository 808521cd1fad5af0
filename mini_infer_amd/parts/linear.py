"""A bias-free linear map `y = x @ W.T` with W in [out, in] layout.

The reference's linears are `F.linear` on the vendor BLAS
(distributed/linear.py:6-14, :167).  Here bfloat16 uses the vendor GEMM too and
float32 runs a hand-written true-float32 kernel.  Several checkpoint tensors can
be stacked along the output axis at load (q|k|v, gate|up) so one product serves
them all (distributed/linear.py:237-249 merges q, k, v the same way).
"""

from __future__ import annotations

import torch

from mini_infer_amd import ops
from mini_infer_amd.parts.base import ParamSpec, Part, TensorGetter


class Linear(Part):
    graph_safe = True

    def __init__(
        self,
        in_features: int,
        out_features: list[int] | int,
        names: list[str] | str,
        dtype: torch.dtype,
        device,
    ) -> None:
        super().__init__(dtype, device)
        self.in_features = in_features
        self.out_splits = [out_features] if isinstance(out_features, int) else list(out_features)
        self.names = [names] if isinstance(names, str) else list(names)
        if len(self.out_splits) != len(self.names):
            raise ValueError("one name per stacked output block")
        self.out_features = sum(self.out_splits)
        self.weight: torch.Tensor | None = None

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        return {
            prefix + name + ".weight": ParamSpec((rows, self.in_features))
            for name, rows in zip(self.names, self.out_splits)
        }

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        blocks = [get(prefix + name + ".weight") for name in self.names]
        self.weight = (blocks[0] if len(blocks) == 1 else torch.cat(blocks, dim=0)).contiguous()

    def forward(self, x: torch.Tensor, partial_ok: bool = False):
        """`x @ weight.T`; with `partial_ok` possibly as `ops.PartialSums` for a norm to add up."""
        assert self.weight is not None, "Linear used before its weight was loaded"
        return ops.linear(x, self.weight, partial_ok=partial_ok)
