"""Engine knobs: cache size, page size, batch limits, compute dtype, seed.

Names follow the reference's constructor arguments where it has them:
`num_blocks` and `block_size` (engine/model_runner.py:27-28, :84-100),
`max_concurrent`, `decode_headroom_blocks`, `chunk_size`, `async_sampling` and
`trace_out` (scheduler/continuous_scheduler.py:144-177).  `max_num_batched_tokens`
is the token budget of one step, which the reference does not have; `seed` is the
base of the per-request sampling seeds.

`ModelRunner.from_pretrained(..., engine=cfg)`, `ContinuousScheduler.from_config(runner,
cfg)`, `LLM` and the command line are all built from one `EngineConfig`.
"""

from __future__ import annotations

import dataclasses

DEFAULT_NUM_BLOCKS = 1024
DEFAULT_BLOCK_SIZE = 16
DEFAULT_MAX_CONCURRENT = 16
DEFAULT_MAX_NUM_BATCHED_TOKENS = 2048
DEFAULT_CHUNK_SIZE = 256
DEFAULT_DECODE_HEADROOM_BLOCKS = 8

_DTYPES = ("bfloat16", "float32")


@dataclasses.dataclass(frozen=True)
class EngineConfig:
    num_blocks: int = DEFAULT_NUM_BLOCKS
    block_size: int = DEFAULT_BLOCK_SIZE
    max_concurrent: int = DEFAULT_MAX_CONCURRENT
    max_num_batched_tokens: int = DEFAULT_MAX_NUM_BATCHED_TOKENS
    chunk_size: int = DEFAULT_CHUNK_SIZE
    decode_headroom_blocks: int = DEFAULT_DECODE_HEADROOM_BLOCKS
    dtype: str = "bfloat16"
    device: str = "cuda:0"
    seed: int = 0
    cuda_graph: bool = True
    async_sampling: bool | None = None  # None: on where the runner and the sampler allow it
    trace_out: str | None = None

    def __post_init__(self) -> None:
        if self.dtype not in _DTYPES:
            raise ValueError(f"dtype must be one of {_DTYPES}, got {self.dtype!r}")
        for name in ("num_blocks", "block_size", "max_concurrent", "max_num_batched_tokens", "chunk_size"):
            if getattr(self, name) <= 0:
                raise ValueError(f"{name} must be positive, got {getattr(self, name)}")
        if self.decode_headroom_blocks < 0:
            raise ValueError(f"decode_headroom_blocks must be >= 0, got {self.decode_headroom_blocks}")
        if not 0 <= self.seed < 2**64:
            raise ValueError(f"seed must fit 64 unsigned bits, got {self.seed}")
