"""Random weights: writes a model folder (config.json + model.safetensors) from a
configuration and a seed.

The reference has no such mode in the library; its tests seed torch and fill
the parameters (tests/unit/models/llama/test_llama_rope_scaling.py:79-96).  Here
the values come from NumPy's PCG64 stream in the sorted order of tensor names,
so any program can reproduce them from (config, seed) alone: linear and
embedding tensors N(0, std), norm weights 1 + N(0, norm_jitter).
"""

from __future__ import annotations

import json
from pathlib import Path
from typing import Any

import numpy as np
import torch
from safetensors.torch import save_file

from mini_infer_amd.parts.base import ParamSpec


def random_tensors(
    specs: dict[str, ParamSpec],
    seed: int,
    *,
    std: float = 0.02,
    norm_jitter: float = 0.1,
    dtype: torch.dtype = torch.bfloat16,
) -> dict[str, torch.Tensor]:
    rng = np.random.Generator(np.random.PCG64(seed))
    out: dict[str, torch.Tensor] = {}
    for name in sorted(specs):
        spec = specs[name]
        values = rng.standard_normal(spec.shape, dtype=np.float32)
        if spec.init == "norm_weight":
            values = 1.0 + norm_jitter * values
        elif spec.init == "normal":
            values = std * values
        else:
            raise ValueError(f"{name}: unknown init {spec.init!r}")
        tensor = torch.from_numpy(np.ascontiguousarray(values, dtype=np.float32))
        store = torch.float32 if spec.dtype == "float32" else dtype
        out[name] = tensor.to(store)
    return out


def write_random_model(
    raw_config: dict[str, Any],
    seed: int,
    out_dir: str | Path,
    *,
    std: float = 0.02,
    norm_jitter: float = 0.1,
    dtype: str = "bfloat16",
) -> Path:
    """Write `out_dir/config.json` and `out_dir/model.safetensors`; returns `out_dir`.

    `raw_config` holds the architecture's own config.json keys; the model class is
    chosen by `architectures[0]` as everywhere else.
    """
    from mini_infer_amd.models import architecture_for

    store = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
    arch = architecture_for(raw_config)
    model = arch.make_model(arch.parse_config(raw_config), store, "cpu")
    tensors = random_tensors(model.param_specs(), seed, std=std, norm_jitter=norm_jitter, dtype=store)
    out_dir = Path(out_dir)
    out_dir.mkdir(parents=True, exist_ok=True)
    with (out_dir / "config.json").open("w") as handle:
        json.dump(raw_config, handle, indent=2)
    save_file(tensors, str(out_dir / "model.safetensors"))
    return out_dir


def fill_random_on_device(model, seed: int, *, std: float = 0.02, norm_jitter: float = 0.0) -> None:
    """Give `model` random weights generated on its own device, tensor by tensor.

    For sizes whose file would be too large to write (benchmarks at 8B and above).
    The values differ from `random_tensors` (another generator); same distributions.
    """
    specs = model.param_specs()
    generator = torch.Generator(device=model.device)
    order = {name: i for i, name in enumerate(sorted(specs))}

    def get(name: str) -> torch.Tensor:
        spec = specs[name]
        generator.manual_seed(seed * 1_000_003 + order[name])
        values = torch.randn(spec.shape, generator=generator, device=model.device, dtype=torch.float32)
        if spec.init == "norm_weight":
            values = 1.0 + norm_jitter * values
        else:
            values = std * values
        return values.to(torch.float32 if spec.dtype == "float32" else model.dtype)

    model.load_params(get)
