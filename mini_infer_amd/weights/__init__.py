from mini_infer_amd.weights.loader import check_names_and_shapes, load_checkpoint, load_state_dict
from mini_infer_amd.weights.random_init import random_tensors, write_random_model
from mini_infer_amd.weights.safetensors_io import CheckpointReader, shard_paths

__all__ = [
    "CheckpointReader",
    "check_names_and_shapes",
    "load_checkpoint",
    "load_state_dict",
    "random_tensors",
    "shard_paths",
    "write_random_model",
]
