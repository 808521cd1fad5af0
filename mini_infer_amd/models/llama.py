"""Llama as a `ModelSpec`: RMSNorm, rotary GQA attention, SwiGLU, pre-norm blocks.

Tensor names are the checkpoint's own (models/llama/llama.py:98-147 of the
reference: `model.embed_tokens`, `model.layers.N.{input_layernorm,self_attn,
post_attention_layernorm,mlp}`, `model.norm`, `lm_head`).
"""

from __future__ import annotations

import dataclasses

from mini_infer_amd.config.model_config import ModelConfig
from mini_infer_amd.models.spec import Architecture, LayerCall, LayerSpec, ModelSpec
from mini_infer_amd.registry import ARCHITECTURES


def llama_spec(cfg: ModelConfig) -> ModelSpec:
    position = {"kind": "rotary", "head_dim": cfg.head_dim, "theta": cfg.rope_theta}
    if cfg.rope_scaling is not None:
        position["llama3"] = dataclasses.asdict(cfg.rope_scaling)
    norm = {"kind": "rms_norm", "hidden_size": cfg.hidden_size, "eps": cfg.rms_norm_eps}
    block = {
        "kind": "pre_norm",
        "norm": norm,
        "mixer": {
            "kind": "gqa_attention",
            "hidden_size": cfg.hidden_size,
            "num_heads": cfg.num_attention_heads,
            "num_kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim,
            "position": position,
        },
        "feed_forward": {
            "kind": "swiglu",
            "hidden_size": cfg.hidden_size,
            "intermediate_size": cfg.intermediate_size,
            "activation": cfg.hidden_act,
        },
        "names": {
            "mixer_norm": "input_layernorm.",
            "mixer": "self_attn.",
            "ffn_norm": "post_attention_layernorm.",
            "feed_forward": "mlp.",
        },
    }
    layers = [LayerSpec(prefix=f"model.layers.{i}.", block=block) for i in range(cfg.num_hidden_layers)]
    return ModelSpec(
        vocab_size=cfg.vocab_size,
        hidden_size=cfg.hidden_size,
        embedding_name="model.embed_tokens.weight",
        layers=layers,
        order=[LayerCall(i) for i in range(cfg.num_hidden_layers)],
        final_norm=norm,
        final_norm_prefix="model.norm.",
        head_name="lm_head.weight",
        tie_word_embeddings=cfg.tie_word_embeddings,
        max_position_embeddings=cfg.max_position_embeddings,
    )


LLAMA = ARCHITECTURES.register(
    "LlamaForCausalLM",
    Architecture(name="LlamaForCausalLM", parse_config=ModelConfig.from_dict, build_spec=llama_spec),
)
