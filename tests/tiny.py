"""Tiny configurations and model folders for the tests.

The configurations differ in every size and option: layers, width, heads
and groups, head size, feed-forward width, vocabulary, rope base and scaling,
the norms' eps, tied or untied head.  A and B are the two named in the project's
baseline; C adds sizes that no vector width divides; D has the smallest sizes at
which every fast path of the bfloat16 engine runs (weight rows of whole cache
lines read as such, both norms of a layer folded into the neighbouring products,
head size 64 on the matrix-core attention with streamed pages); E and F have head
sizes of 100 and 40, which no 16-byte load divides.  Weights are made here with
NumPy (not with the engine's random mode), rounded to bfloat16 so the float32
and the bfloat16 engine and the plain implementation all read the same numbers.
"""

from __future__ import annotations

import json
from pathlib import Path

import numpy as np
import torch
from safetensors.torch import save_file

TINY_A = {
    "architectures": ["LlamaForCausalLM"],
    "num_hidden_layers": 2,
    "hidden_size": 64,
    "num_attention_heads": 4,
    "num_key_value_heads": 2,
    "head_dim": 16,
    "intermediate_size": 160,
    "vocab_size": 256,
    "rope_theta": 10000.0,
    "rope_scaling": None,
    "rms_norm_eps": 1e-6,
    "tie_word_embeddings": True,
    "max_position_embeddings": 128,
}
TINY_A_BLOCK = 4

TINY_B = {
    "architectures": ["LlamaForCausalLM"],
    "num_hidden_layers": 3,
    "hidden_size": 96,
    "num_attention_heads": 3,
    "num_key_value_heads": 1,
    "head_dim": 32,
    "intermediate_size": 256,
    "vocab_size": 384,
    "rope_theta": 500000.0,
    "rope_scaling": {
        "rope_type": "llama3",
        "factor": 8.0,
        "low_freq_factor": 1.0,
        "high_freq_factor": 4.0,
        "original_max_position_embeddings": 64,
    },
    "rms_norm_eps": 1e-5,
    "tie_word_embeddings": False,
    "max_position_embeddings": 512,
}
TINY_B_BLOCK = 16

TINY_C = {
    "architectures": ["LlamaForCausalLM"],
    "num_hidden_layers": 2,
    "hidden_size": 90,
    "num_attention_heads": 6,
    "num_key_value_heads": 3,
    "head_dim": 48,
    "intermediate_size": 130,
    "vocab_size": 301,
    "rope_parameters": {
        "rope_type": "llama3",
        "rope_theta": 20000.0,
        "factor": 4.0,
        "low_freq_factor": 1.0,
        "high_freq_factor": 2.0,
        "original_max_position_embeddings": 32,
    },
    "rms_norm_eps": 3e-6,
    "tie_word_embeddings": False,
    "max_position_embeddings": 1024,
}
TINY_C_BLOCK = 8

TINY_D = {
    "architectures": ["LlamaForCausalLM"],
    "num_hidden_layers": 2,
    "hidden_size": 512,
    "num_attention_heads": 8,
    "num_key_value_heads": 2,
    "head_dim": 64,
    "intermediate_size": 1024,
    "vocab_size": 333,
    "rope_theta": 100000.0,
    "rope_scaling": {
        "rope_type": "llama3",
        "factor": 16.0,
        "low_freq_factor": 1.0,
        "high_freq_factor": 8.0,
        "original_max_position_embeddings": 48,
    },
    "rms_norm_eps": 2e-5,
    "tie_word_embeddings": True,
    "max_position_embeddings": 2048,
}
TINY_D_BLOCK = 16

# E and F: head sizes that are not a multiple of 16.  E names no `head_dim`: it is
# hidden_size / num_attention_heads = 100, the head size of a 3200-wide model with 32 heads.
TINY_E = {
    "architectures": ["LlamaForCausalLM"],
    "num_hidden_layers": 2,
    "hidden_size": 200,
    "num_attention_heads": 2,
    "num_key_value_heads": 1,
    "intermediate_size": 176,
    "vocab_size": 211,
    "rope_theta": 10000.0,
    "rms_norm_eps": 1e-5,
    "tie_word_embeddings": False,
    "max_position_embeddings": 256,
}
TINY_E_BLOCK = 16

TINY_F = {
    "architectures": ["LlamaForCausalLM"],
    "num_hidden_layers": 3,
    "hidden_size": 160,
    "num_attention_heads": 4,
    "num_key_value_heads": 2,
    "head_dim": 40,
    "intermediate_size": 96,
    "vocab_size": 199,
    "rope_theta": 50000.0,
    "rope_scaling": {
        "rope_type": "llama3",
        "factor": 2.0,
        "low_freq_factor": 1.0,
        "high_freq_factor": 4.0,
        "original_max_position_embeddings": 40,
    },
    "rms_norm_eps": 1e-6,
    "tie_word_embeddings": True,
    "max_position_embeddings": 512,
}
TINY_F_BLOCK = 8

CONFIGS = {"A": (TINY_A, TINY_A_BLOCK), "B": (TINY_B, TINY_B_BLOCK), "C": (TINY_C, TINY_C_BLOCK),
           "D": (TINY_D, TINY_D_BLOCK), "E": (TINY_E, TINY_E_BLOCK), "F": (TINY_F, TINY_F_BLOCK)}


def bf16_round(values: np.ndarray) -> np.ndarray:
    """float32 values rounded to the nearest bfloat16, returned as float32."""
    return torch.from_numpy(np.ascontiguousarray(values, dtype=np.float32)).bfloat16().float().numpy()


def tensor_shapes(cfg: dict) -> dict[str, tuple[int, ...]]:
    h, i, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    d = cfg.get("head_dim") or h // cfg["num_attention_heads"]
    q, kv = cfg["num_attention_heads"] * d, cfg["num_key_value_heads"] * d
    shapes = {"model.embed_tokens.weight": (v, h), "model.norm.weight": (h,)}
    if not cfg.get("tie_word_embeddings", False):
        shapes["lm_head.weight"] = (v, h)
    for n in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{n}."
        shapes[p + "input_layernorm.weight"] = (h,)
        shapes[p + "post_attention_layernorm.weight"] = (h,)
        shapes[p + "self_attn.q_proj.weight"] = (q, h)
        shapes[p + "self_attn.k_proj.weight"] = (kv, h)
        shapes[p + "self_attn.v_proj.weight"] = (kv, h)
        shapes[p + "self_attn.o_proj.weight"] = (h, q)
        shapes[p + "mlp.gate_proj.weight"] = (i, h)
        shapes[p + "mlp.up_proj.weight"] = (i, h)
        shapes[p + "mlp.down_proj.weight"] = (h, i)
    return shapes


def make_weights(cfg: dict, seed: int, *, qk_gain: float = 2.0) -> dict[str, np.ndarray]:
    """Random weights with activations of order one and peaked attention.

    Linear maps N(0, 1/fan_in), embedding N(0, 1), norm weights U(0.5, 1.5); q and
    k projections are scaled by `qk_gain` so scores are large enough that a wrong
    rotation or a missing key moves the logits.  Values are bfloat16-exact.
    """
    rng = np.random.default_rng(seed)
    out: dict[str, np.ndarray] = {}
    for name, shape in sorted(tensor_shapes(cfg).items()):
        if name.endswith("layernorm.weight") or name == "model.norm.weight":
            values = rng.uniform(0.5, 1.5, size=shape)
        elif name == "model.embed_tokens.weight":
            values = rng.standard_normal(shape)
        else:
            values = rng.standard_normal(shape) / np.sqrt(shape[1])
            if "q_proj" in name or "k_proj" in name:
                values = values * qk_gain
        out[name] = bf16_round(values.astype(np.float32))
    return out


def write_model_dir(path: Path, cfg: dict, weights: dict[str, np.ndarray], dtype=torch.bfloat16) -> Path:
    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    with (path / "config.json").open("w") as handle:
        json.dump(cfg, handle)
    tensors = {k: torch.from_numpy(np.ascontiguousarray(v)).to(dtype) for k, v in weights.items()}
    save_file(tensors, str(path / "model.safetensors"))
    return path


def random_tokens(cfg: dict, length: int, seed: int) -> list[int]:
    rng = np.random.default_rng(seed)
    return rng.integers(0, cfg["vocab_size"], size=length).tolist()
