"""`LLM(...).generate(...)`: the short way from a model folder to generated tokens.

It is the reference's quick-start (README.md:106-131: `ModelRunner.from_pretrained`
+ `ContinuousScheduler` + `Request`) in one object, driven synchronously.
"""

from __future__ import annotations

from pathlib import Path
from typing import Sequence

from mini_infer_amd.config import (
    DEFAULT_BLOCK_SIZE,
    DEFAULT_CHUNK_SIZE,
    DEFAULT_DECODE_HEADROOM_BLOCKS,
    DEFAULT_MAX_CONCURRENT,
    DEFAULT_MAX_NUM_BATCHED_TOKENS,
    DEFAULT_NUM_BLOCKS,
    EngineConfig,
    read_config_json,
)
from mini_infer_amd.engine.model_runner import ModelRunner
from mini_infer_amd.engine.request import GenerationResult, Request
from mini_infer_amd.engine.scheduler import ContinuousScheduler
from mini_infer_amd.engine.tokenizer import Tokenizer
from mini_infer_amd.sampling.params import SamplingParams


class LLM:
    def __init__(
        self,
        model: str | Path,
        *,
        engine: EngineConfig | None = None,
        dtype: str = "bfloat16",
        device: str = "cuda:0",
        num_blocks: int = DEFAULT_NUM_BLOCKS,
        block_size: int = DEFAULT_BLOCK_SIZE,
        max_concurrent: int = DEFAULT_MAX_CONCURRENT,
        max_num_batched_tokens: int = DEFAULT_MAX_NUM_BATCHED_TOKENS,
        chunk_size: int = DEFAULT_CHUNK_SIZE,
        decode_headroom_blocks: int = DEFAULT_DECODE_HEADROOM_BLOCKS,
        seed: int = 0,
        async_sampling: bool | None = None,
        trace_out: str | None = None,
    ) -> None:
        """The engine's knobs come as one `EngineConfig` (`engine=`) or as the keyword
        arguments of the same names, from which one is made (and so checked) here."""
        if engine is None:
            engine = EngineConfig(
                num_blocks=num_blocks, block_size=block_size, max_concurrent=max_concurrent,
                max_num_batched_tokens=max_num_batched_tokens, chunk_size=chunk_size,
                decode_headroom_blocks=decode_headroom_blocks, dtype=dtype, device=device, seed=seed,
                async_sampling=async_sampling, trace_out=trace_out,
            )
        self.engine_config = engine
        self.runner = ModelRunner.from_pretrained(model, engine=engine)
        raw = read_config_json(model)
        self.tokenizer = Tokenizer.from_pretrained(model)
        self.scheduler = ContinuousScheduler.from_config(
            self.runner, engine, eos_token_id=raw.get("eos_token_id"), tokenizer=self.tokenizer
        )

    def generate(
        self,
        prompts: Sequence[str | Sequence[int]],
        sampling_params: SamplingParams | Sequence[SamplingParams] | None = None,
        max_tokens: int = 16,
    ) -> list[GenerationResult]:
        """One result per prompt (text or token ids), in order."""
        if sampling_params is None:
            sampling_params = SamplingParams()
        if isinstance(sampling_params, SamplingParams):
            sampling_params = [sampling_params] * len(prompts)
        if len(sampling_params) != len(prompts):
            raise ValueError("one SamplingParams per prompt (or one for all)")
        requests = [Request(p, sp, max_tokens) for p, sp in zip(prompts, sampling_params)]
        results = self.scheduler.run_all(requests)
        self.scheduler.write_trace()
        return results
