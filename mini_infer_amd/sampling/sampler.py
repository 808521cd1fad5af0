"""Batched next-token choice on the device.

One kernel call per step for all rows: greedy rows take the first maximum,
sampling rows apply temperature, top-k and top-p and draw (the reference's
`sample_tokens`, engine/sampler.py:49-90).  Row i's draw is keyed by
(seed_i, draw_index_i): the same request gives the same tokens alone or in any batch.
"""

from __future__ import annotations

from typing import Sequence

import numpy as np
import torch

from mini_infer_amd import ops
from mini_infer_amd.sampling.params import SamplingParams


def _as_i32(values: np.ndarray) -> np.ndarray:
    """Unsigned 32-bit patterns carried in int32 (torch has no uint32 arithmetic needs here)."""
    return values.astype(np.uint32).view(np.int32)


def sample_tokens(
    logits: torch.Tensor,
    params: Sequence[SamplingParams],
    seeds: Sequence[int],
    draw_indices: Sequence[int],
) -> torch.Tensor:
    """One id per row of `logits` [B, V] (float32 or bfloat16), as an int32 device tensor."""
    rows = logits.shape[0]
    if logits.dim() != 2 or rows != len(params) or rows != len(seeds) or rows != len(draw_indices):
        raise ValueError(
            f"logits must be (batch, vocab) with one params, seed and draw index per row; got "
            f"{tuple(logits.shape)} for {len(params)} params"
        )
    vocab = logits.shape[1]
    settings = np.empty((6, rows), dtype=np.int32)
    settings[0] = np.array([p.temperature for p in params], dtype=np.float32).view(np.int32)
    settings[1] = np.array([p.top_k if 0 < p.top_k < vocab else 0 for p in params], dtype=np.int32)
    settings[2] = np.array([p.top_p for p in params], dtype=np.float32).view(np.int32)
    seeds64 = np.array([s & 0xFFFFFFFFFFFFFFFF for s in seeds], dtype=np.uint64)
    settings[3] = _as_i32(seeds64 & np.uint64(0xFFFFFFFF))
    settings[4] = _as_i32(seeds64 >> np.uint64(32))
    settings[5] = _as_i32(np.array(draw_indices, dtype=np.uint64) & np.uint64(0xFFFFFFFF))
    staged = torch.from_numpy(settings).pin_memory().to(logits.device, non_blocking=True)
    return ops.sample(
        logits,
        staged[0].view(torch.float32),
        staged[1],
        staged[2].view(torch.float32),
        staged[3],
        staged[4],
        staged[5],
    )


def sample_from_slots(logits: torch.Tensor, row_slots: torch.Tensor, slot_table: torch.Tensor) -> torch.Tensor:
    """One id per row of `logits` as an int32 device tensor, every row's settings, seed and draw
    index read on the device from its request's state slot (`row_slots[b]` of `slot_table`); the
    kernel advances the draw index, so nothing about sampling travels from the host per step."""
    if logits.dim() != 2 or row_slots.numel() != logits.shape[0]:
        raise ValueError(
            f"logits must be (batch, vocab) with one slot id per row; got {tuple(logits.shape)} and {row_slots.numel()} slots"
        )
    return ops.sample_slots(logits, row_slots, slot_table)


def sample_batch(
    logits: torch.Tensor,
    params: Sequence[SamplingParams],
    seeds: Sequence[int],
    draw_indices: Sequence[int],
) -> list[int]:
    """`sample_tokens` with one copy of the ids to the host."""
    return sample_tokens(logits, params, seeds, draw_indices).tolist()
