"""Rotary position encoding: the inverse-frequency table and how dims are paired.

`inv_freq = theta^(-2j/D)` in float32 (models/blocks/rope.py:343-346 of the
reference), optionally rescaled the llama3 way (rope.py:200-225).  The table
stays float32 whatever the compute dtype (rope.py:368-390), and the angles
`position * inv_freq` and their cos/sin are float32 too.

A mixer asks this part for the cos/sin tables of a step (`rotary(ctx)`); they are
computed once per step and shared by all layers that use the same encoding.
"""

from __future__ import annotations

import math

import torch

from mini_infer_amd import ops
from mini_infer_amd.parts.base import PositionEncoding, RotaryTables, StepContext
from mini_infer_amd.registry import register_position_encoding


def default_inv_freq(rotary_dim: int, theta: float) -> torch.Tensor:
    exponent = torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim
    return 1.0 / (theta**exponent)


def llama3_inv_freq(
    inv_freq: torch.Tensor,
    factor: float,
    low_freq_factor: float,
    high_freq_factor: float,
    original_max_position_embeddings: int,
) -> torch.Tensor:
    """Long wavelengths divided by `factor`, short ones kept, the band between blended."""
    old_len = original_max_position_embeddings
    low_wavelen = old_len / low_freq_factor
    high_wavelen = old_len / high_freq_factor
    wavelen = 2 * math.pi / inv_freq
    scaled = torch.where(wavelen > low_wavelen, inv_freq / factor, inv_freq)
    smooth = (old_len / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
    smoothed = (1 - smooth) * scaled / factor + smooth * scaled
    medium = ~(wavelen < high_wavelen) & ~(wavelen > low_wavelen)
    return torch.where(medium, smoothed, scaled)


class RotaryPosition(PositionEncoding):
    """Rotation of the first `rotary_dim` dims of each head.

    `interleaved=False` pairs dim j with j + rotary_dim/2 (the Llama way,
    rope.py:411-416); `interleaved=True` pairs 2j with 2j+1.
    """

    def __init__(
        self,
        head_dim: int,
        theta: float,
        dtype: torch.dtype,
        device,
        *,
        rotary_dim: int | None = None,
        interleaved: bool = False,
        llama3: dict | None = None,
    ) -> None:
        super().__init__(dtype, device)
        self.head_dim = head_dim
        self.rotary_dim = head_dim if rotary_dim is None else int(rotary_dim)
        if self.rotary_dim % 2 != 0 or not 0 < self.rotary_dim <= head_dim:
            raise ValueError(f"rotary_dim={self.rotary_dim} must be even and within head_dim={head_dim}")
        self.interleaved = bool(interleaved)
        table = default_inv_freq(self.rotary_dim, float(theta))
        if llama3 is not None:
            table = llama3_inv_freq(
                table,
                float(llama3["factor"]),
                float(llama3["low_freq_factor"]),
                float(llama3["high_freq_factor"]),
                int(llama3["original_max_position_embeddings"]),
            )
        self.inv_freq_host = table.to(torch.float32)
        self._inv_freq_device: torch.Tensor | None = None

    @property
    def inv_freq(self) -> torch.Tensor:
        if self._inv_freq_device is None:
            self._inv_freq_device = self.inv_freq_host.to(self.device).contiguous()
        return self._inv_freq_device

    def tables(self, ctx: StepContext) -> tuple[torch.Tensor, torch.Tensor]:
        """cos, sin [T, rotary_dim/2] float32 for this step's positions (made once a step)."""
        key = ("rotary_tables", id(self))
        if key not in ctx.shared:
            ctx.shared[key] = ops.rope_table(ctx.positions, self.inv_freq)
        return ctx.shared[key]

    def rotary_layout(self) -> tuple[int, bool]:
        return self.rotary_dim, self.interleaved

    def rotary(self, ctx: StepContext) -> RotaryTables:
        cos, sin = self.tables(ctx)
        return RotaryTables(cos, sin, self.rotary_dim, self.interleaved)


@register_position_encoding("rotary")
def build_rotary(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> RotaryPosition:
    return RotaryPosition(
        int(desc["head_dim"]),
        float(desc["theta"]),
        dtype,
        device,
        rotary_dim=desc.get("rotary_dim"),
        interleaved=bool(desc.get("interleaved", False)),
        llama3=desc.get("llama3"),
    )
