"""Typed model configuration read from an architecture's own config.json keys.

Keys, defaults and refusals follow the reference's `LlamaConfig.from_hf`
(models/llama/llama.py:40-95) and `read_rope_parameters`
(models/blocks/rope.py:228-269).  Nothing here knows a model size: every
number comes from the file.
"""

from __future__ import annotations

import dataclasses
import json
from pathlib import Path
from typing import Any

from mini_infer_amd.exceptions import ConfigError


@dataclasses.dataclass(frozen=True)
class Llama3RopeScaling:
    """`rope_type: "llama3"` parameters (models/blocks/rope.py:171-197)."""

    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int

    def __post_init__(self) -> None:
        if self.factor <= 0:
            raise ConfigError(f"llama3 rope factor must be positive, got {self.factor}")
        if self.high_freq_factor <= self.low_freq_factor:
            raise ConfigError(
                "llama3 rope needs high_freq_factor > low_freq_factor, got "
                f"{self.high_freq_factor} <= {self.low_freq_factor}"
            )
        if self.original_max_position_embeddings <= 0:
            raise ConfigError(
                "llama3 rope original_max_position_embeddings must be positive, got "
                f"{self.original_max_position_embeddings}"
            )


def read_rope_parameters(raw: dict[str, Any]) -> tuple[float, Llama3RopeScaling | None]:
    """`(rope_theta, llama3 scaling or None)` from raw config.json keys.

    The dict lives under `rope_parameters` (newer files, theta inside) or
    `rope_scaling` (older files, may be null, theta at top level); the type is
    under `rope_type` or `type`.  Any type but "default" and "llama3" raises
    `NotImplementedError` (models/blocks/rope.py:242-269).
    """
    params = dict(raw.get("rope_parameters") or raw.get("rope_scaling") or {})
    if "rope_theta" in params:
        theta = float(params["rope_theta"])
    else:
        theta = float(raw.get("rope_theta") or 10000.0)
    kind = params.get("rope_type") or params.get("type") or "default"
    if kind == "default":
        return theta, None
    if kind == "llama3":
        try:
            scaling = Llama3RopeScaling(
                factor=float(params["factor"]),
                low_freq_factor=float(params["low_freq_factor"]),
                high_freq_factor=float(params["high_freq_factor"]),
                original_max_position_embeddings=int(params["original_max_position_embeddings"]),
            )
        except KeyError as missing:
            raise ConfigError(
                f"llama3 rope parameters are missing {missing}; got {sorted(params)}"
            ) from None
        return theta, scaling
    raise NotImplementedError(
        f"rope_type={kind!r} is not supported; only 'default' and 'llama3' are"
    )


_REQUIRED = (
    "vocab_size",
    "hidden_size",
    "intermediate_size",
    "num_hidden_layers",
    "num_attention_heads",
    "num_key_value_heads",
    "rms_norm_eps",
)


@dataclasses.dataclass(frozen=True)
class ModelConfig:
    """A Llama-shaped decoder's numbers, all from config.json."""

    architecture: str
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool
    max_position_embeddings: int | None = None
    rope_scaling: Llama3RopeScaling | None = None
    hidden_act: str = "silu"

    def __post_init__(self) -> None:
        for name in (
            "vocab_size",
            "hidden_size",
            "intermediate_size",
            "num_hidden_layers",
            "num_attention_heads",
            "num_key_value_heads",
            "head_dim",
        ):
            if int(getattr(self, name)) <= 0:
                raise ConfigError(f"{name} must be positive, got {getattr(self, name)}")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError(
                f"num_attention_heads={self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads={self.num_key_value_heads}"
            )
        if self.head_dim % 2 != 0:
            raise ConfigError(f"head_dim must be even for rotary positions, got {self.head_dim}")
        if self.rms_norm_eps <= 0:
            raise ConfigError(f"rms_norm_eps must be positive, got {self.rms_norm_eps}")
        if self.hidden_act != "silu":
            raise NotImplementedError(f"hidden_act={self.hidden_act!r}; only 'silu' is built")

    # -- reading ------------------------------------------------------------

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> ModelConfig:
        architectures = raw.get("architectures") or []
        if not architectures:
            raise ConfigError("config.json has no `architectures`; cannot choose a model")
        missing = [k for k in _REQUIRED if raw.get(k) is None]
        if missing:
            raise ConfigError(f"config.json is missing {missing}")
        if raw.get("attention_bias", False):
            raise NotImplementedError("attention_bias=true is not supported (biased q/k/v)")
        if raw.get("mlp_bias", False):
            raise NotImplementedError("mlp_bias=true is not supported (biased feed-forward)")
        head_dim = raw.get("head_dim") or (raw["hidden_size"] // raw["num_attention_heads"])
        theta, scaling = read_rope_parameters(raw)
        return cls(
            architecture=str(architectures[0]),
            vocab_size=int(raw["vocab_size"]),
            hidden_size=int(raw["hidden_size"]),
            intermediate_size=int(raw["intermediate_size"]),
            num_hidden_layers=int(raw["num_hidden_layers"]),
            num_attention_heads=int(raw["num_attention_heads"]),
            num_key_value_heads=int(raw["num_key_value_heads"]),
            head_dim=int(head_dim),
            rms_norm_eps=float(raw["rms_norm_eps"]),
            rope_theta=theta,
            tie_word_embeddings=bool(raw.get("tie_word_embeddings", False)),
            max_position_embeddings=(
                int(raw["max_position_embeddings"])
                if raw.get("max_position_embeddings") is not None
                else None
            ),
            rope_scaling=scaling,
            hidden_act=str(raw.get("hidden_act", "silu")),
        )

    @classmethod
    def from_json(cls, path: str | Path) -> ModelConfig:
        return cls.from_dict(read_config_json(path))

    # -- writing (for the random-weights mode) -------------------------------

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {
            "architectures": [self.architecture],
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": self.hidden_act,
            "attention_bias": False,
            "mlp_bias": False,
        }
        if self.max_position_embeddings is not None:
            out["max_position_embeddings"] = self.max_position_embeddings
        if self.rope_scaling is None:
            out["rope_scaling"] = None
        else:
            out["rope_scaling"] = {
                "rope_type": "llama3",
                **dataclasses.asdict(self.rope_scaling),
            }
        return out


def read_config_json(path: str | Path) -> dict[str, Any]:
    """The raw keys of `DIR/config.json` (or of the file itself)."""
    path = Path(path)
    if path.is_dir():
        path = path / "config.json"
    if not path.exists():
        raise FileNotFoundError(f"no config.json at {path}")
    with path.open() as handle:
        raw = json.load(handle)
    if not isinstance(raw, dict):
        raise ConfigError(f"{path} does not hold a JSON object")
    return raw
