"""Engine knobs: cache size, page size, batch limits, compute dtype.

Names follow the reference's constructor arguments where it has them:
`num_blocks` and `block_size` (engine/model_runner.py:27-28, :84-100),
`max_concurrent`, `decode_headroom_blocks` and `chunk_size`
(scheduler/continuous_scheduler.py:144-177).  `max_num_batched_tokens` is the
token budget of one step, which the reference does not have.
"""

from __future__ import annotations

import dataclasses

DEFAULT_NUM_BLOCKS = 1024
DEFAULT_BLOCK_SIZE = 16

_DTYPES = ("bfloat16", "float32")


@dataclasses.dataclass(frozen=True)
class EngineConfig:
    num_blocks: int = DEFAULT_NUM_BLOCKS
    block_size: int = DEFAULT_BLOCK_SIZE
    max_concurrent: int = 16
    max_num_batched_tokens: int = 2048
    dtype: str = "bfloat16"
    device: str = "cuda:0"

    def __post_init__(self) -> None:
        if self.dtype not in _DTYPES:
            raise ValueError(f"dtype must be one of {_DTYPES}, got {self.dtype!r}")
        if self.num_blocks <= 0:
            raise ValueError(f"num_blocks must be positive, got {self.num_blocks}")
        if self.block_size <= 0:
            raise ValueError(f"block_size must be positive, got {self.block_size}")
        if self.max_concurrent <= 0:
            raise ValueError(f"max_concurrent must be positive, got {self.max_concurrent}")
        if self.max_num_batched_tokens <= 0:
            raise ValueError(
                f"max_num_batched_tokens must be positive, got {self.max_num_batched_tokens}"
            )
