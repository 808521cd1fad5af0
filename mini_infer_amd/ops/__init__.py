"""The hand-written HIP kernels of the engine, as functions on torch tensors."""

from mini_infer_amd.ops.kernels import (
    add_rmsnorm,
    attention_splits,
    embed_gather,
    gemm_f32,
    gemm_skinny_bf16,
    linear_swiglu,
    linear,
    mfma_attention_supported,
    paged_attention,
    qkv_rope_write,
    qkv_rope_write_takes,
    rope_kv_write,
    rope_table,
    sample,
    silu_mul,
    take_device_tokens,
)

__all__ = [
    "add_rmsnorm",
    "attention_splits",
    "embed_gather",
    "gemm_f32",
    "gemm_skinny_bf16",
    "linear_swiglu",
    "linear",
    "mfma_attention_supported",
    "paged_attention",
    "qkv_rope_write",
    "qkv_rope_write_takes",
    "rope_kv_write",
    "rope_table",
    "sample",
    "silu_mul",
    "take_device_tokens",
]
