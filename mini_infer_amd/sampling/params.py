"""Sampling options of a request.

`temperature`, `top_k` and `top_p` have the reference's names, defaults and
checks (engine/sampler.py:7-21): temperature 0 is greedy; top_k 0 and top_p 1 are
off.  `seed` and `ignore_eos` are additions: a request's draws come from a
counter-based generator keyed by its seed, so they do not depend on what else is
in the batch; `ignore_eos` keeps generating past the end-of-sequence token
(benchmarks with random weights).
"""

from __future__ import annotations

import dataclasses


@dataclasses.dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0
    top_k: int = 0
    top_p: float = 1.0
    seed: int | None = None
    ignore_eos: bool = False

    def __post_init__(self) -> None:
        if self.temperature < 0:
            raise ValueError(f"temperature must be >= 0, got {self.temperature}")
        if self.top_k < 0:
            raise ValueError(f"top_k must be >= 0, got {self.top_k}")
        if not 0.0 <= self.top_p <= 1.0:
            raise ValueError(f"top_p must be in [0, 1], got {self.top_p}")
        if self.seed is not None and not 0 <= self.seed < 2**64:
            raise ValueError(f"seed must fit 64 unsigned bits, got {self.seed}")
