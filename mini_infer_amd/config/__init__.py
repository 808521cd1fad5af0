from mini_infer_amd.config.engine_config import (
    DEFAULT_BLOCK_SIZE,
    DEFAULT_CHUNK_SIZE,
    DEFAULT_DECODE_HEADROOM_BLOCKS,
    DEFAULT_MAX_CONCURRENT,
    DEFAULT_MAX_NUM_BATCHED_TOKENS,
    DEFAULT_NUM_BLOCKS,
    EngineConfig,
)
from mini_infer_amd.config.model_config import (
    Llama3RopeScaling,
    ModelConfig,
    read_config_json,
    read_rope_parameters,
)

__all__ = [
    "DEFAULT_BLOCK_SIZE",
    "DEFAULT_CHUNK_SIZE",
    "DEFAULT_DECODE_HEADROOM_BLOCKS",
    "DEFAULT_MAX_CONCURRENT",
    "DEFAULT_MAX_NUM_BATCHED_TOKENS",
    "DEFAULT_NUM_BLOCKS",
    "EngineConfig",
    "Llama3RopeScaling",
    "ModelConfig",
    "read_config_json",
    "read_rope_parameters",
]
