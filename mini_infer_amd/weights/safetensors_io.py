"""Finding and reading safetensors checkpoints by tensor name.

Layouts as in the reference's loader (models/loader.py:140-151, :188-215): a
single `model.safetensors`, or shards listed in `model.safetensors.index.json`.
Tensors are read one at a time through `safe_open`, so a large checkpoint never
needs a full host copy.
"""

from __future__ import annotations

import json
from pathlib import Path

import torch
from safetensors import safe_open


def shard_paths(model_dir: str | Path) -> list[Path]:
    model_dir = Path(model_dir)
    index = model_dir / "model.safetensors.index.json"
    if index.exists():
        with index.open() as handle:
            weight_map = json.load(handle)["weight_map"]
        return [model_dir / shard for shard in sorted(set(weight_map.values()))]
    single = model_dir / "model.safetensors"
    if not single.exists():
        raise FileNotFoundError(f"no model.safetensors or model.safetensors.index.json under {model_dir}")
    return [single]


class CheckpointReader:
    """Name -> (shape, dtype) of every tensor in a checkpoint, and reads by name."""

    def __init__(self, model_dir: str | Path) -> None:
        self.paths = shard_paths(model_dir)
        self._where: dict[str, Path] = {}
        self.shapes: dict[str, tuple[int, ...]] = {}
        self.dtypes: dict[str, str] = {}
        for path in self.paths:
            with safe_open(str(path), framework="pt", device="cpu") as handle:
                for name in handle.keys():  # noqa: SIM118
                    self._where[name] = path
                    view = handle.get_slice(name)
                    self.shapes[name] = tuple(view.get_shape())
                    self.dtypes[name] = str(view.get_dtype())

    def names(self) -> list[str]:
        return sorted(self._where)

    def read(self, name: str) -> torch.Tensor:
        with safe_open(str(self._where[name]), framework="pt", device="cpu") as handle:
            return handle.get_tensor(name)
