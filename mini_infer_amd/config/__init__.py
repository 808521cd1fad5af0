from mini_infer_amd.config.engine_config import (
    DEFAULT_BLOCK_SIZE,
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
    "DEFAULT_NUM_BLOCKS",
    "EngineConfig",
    "Llama3RopeScaling",
    "ModelConfig",
    "read_config_json",
    "read_rope_parameters",
]
