"""Loading a checkpoint into a model by tensor name.

Rules (the reference's are in models/loader.py:73-89 and
distributed/loader.py:101-108, :168-173, :202-205; models/llama/llama.py:200-207):
  * the model states the tensors it needs (`param_specs`); the file must hold
    exactly those (plus names the model declares optional, e.g. `lm_head.weight`
    beside tied embeddings);
  * missing names, unexpected names and wrong shapes are all reported in ONE
    `WeightLoadError`;
  * floating tensors are cast to the engine's dtype, except that a parameter
    declared "float32" stays 32-bit and integer tables are kept as int32.
"""

from __future__ import annotations

from pathlib import Path

import torch

from mini_infer_amd.exceptions import WeightLoadError
from mini_infer_amd.parts.base import ParamSpec
from mini_infer_amd.weights.safetensors_io import CheckpointReader


def check_names_and_shapes(
    specs: dict[str, ParamSpec],
    optional: set[str],
    found_shapes: dict[str, tuple[int, ...]],
) -> None:
    missing = sorted(name for name in specs if name not in found_shapes)
    unexpected = sorted(name for name in found_shapes if name not in specs and name not in optional)
    wrong = sorted(
        (name, tuple(found_shapes[name]), tuple(spec.shape))
        for name, spec in specs.items()
        if name in found_shapes and tuple(found_shapes[name]) != tuple(spec.shape)
    )
    if missing or unexpected or wrong:
        lines = ["weight load mismatch:"]
        lines.append(f"  missing={missing}")
        lines.append(f"  unexpected={unexpected}")
        lines.append(
            "  wrong_shape=["
            + ", ".join(f"{n}: found {f}, expected {e}" for n, f, e in wrong)
            + "]"
        )
        raise WeightLoadError("\n".join(lines))


def target_dtype(spec: ParamSpec, stored: torch.dtype, compute: torch.dtype) -> torch.dtype:
    if spec.dtype == "float32":
        return torch.float32
    if spec.dtype == "int32" or not stored.is_floating_point:
        return torch.int32
    return compute


def load_checkpoint(model, model_dir: str | Path) -> None:
    """Read `model_dir`'s safetensors into `model` (anything with `param_specs`,
    `optional_names`, `load_params`, `dtype`, `device`)."""
    reader = CheckpointReader(model_dir)
    specs = model.param_specs()
    check_names_and_shapes(specs, model.optional_names(), reader.shapes)

    def get(name: str) -> torch.Tensor:
        stored = reader.read(name)
        wanted = target_dtype(specs[name], stored.dtype, model.dtype)
        return stored.to(device=model.device, dtype=wanted)

    model.load_params(get)


def load_state_dict(model, tensors: dict[str, torch.Tensor]) -> None:
    """The same checks and casts for tensors already in memory."""
    specs = model.param_specs()
    check_names_and_shapes(specs, model.optional_names(), {k: tuple(v.shape) for k, v in tensors.items()})

    def get(name: str) -> torch.Tensor:
        stored = tensors[name]
        wanted = target_dtype(specs[name], stored.dtype, model.dtype)
        return stored.to(device=model.device, dtype=wanted)

    model.load_params(get)
