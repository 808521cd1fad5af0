"""The plain Llama decoder of `plain_llama.py` once more, in torch float64, for inputs too
large for NumPy on a CPU (thousands of tokens at the widths of an 8B model).

Same formulas, same order, whole sequences, no cache; it shares no code with the engine
and uses no kernel of it (torch's own float64 products and elementwise routines only,
on whatever device it is given).  `tests/test_plain_reference.py` pins it to the NumPy
implementation on the tiny configurations, so everything that fixes that one fixes this one.

Paths cited are relative to the reference's `src/mini_infer/`.
"""

from __future__ import annotations

import math

import numpy as np
import torch

import plain_llama

ACC = torch.float64


def _keep(x: torch.Tensor) -> torch.Tensor:
    return x


def bf16_round(x: torch.Tensor) -> torch.Tensor:
    """Values rounded to the nearest bfloat16, as float64."""
    return x.to(torch.float32).to(torch.bfloat16).to(ACC)


def rope_tables(positions: torch.Tensor, inv_freq: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """models/blocks/rope.py:392-408: float32 angles `pos * inv_freq`, halves repeated."""
    freqs = positions.to(torch.float32)[:, None] * inv_freq.to(torch.float32)[None, :]
    emb = torch.cat([freqs, freqs], dim=-1).to(ACC)
    return torch.cos(emb), torch.sin(emb)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """models/blocks/rope.py:411-431: `x*cos + rotate_half(x)*sin`, x [T, heads, D]."""
    half = x.shape[-1] // 2
    rotated = torch.cat([-x[..., half:], x[..., :half]], dim=-1)
    return x * cos[:, None, :] + rotated * sin[:, None, :]


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """models/blocks/rmsnorm.py:81-93."""
    variance = (x * x).mean(dim=-1, keepdim=True)
    return weight * (x / torch.sqrt(variance + eps))


def swiglu(x, w_gate, w_up, w_down, store=_keep):
    """models/blocks/swiglu.py:44-46, activations.py:36-45."""
    gate = store(x @ w_gate.T)
    up = store(x @ w_up.T)
    return store(store(gate / (1.0 + torch.exp(-gate)) * up) @ w_down.T)


def causal_attention(q, k, v, scale: float, window: int | None = None) -> torch.Tensor:
    """cache/packed_attention.py:296-338: q [Tq, Hq, D], k and v [Tk, Hkv, D], the queries are
    the last Tq positions; head h reads key/value head h // (Hq/Hkv).  One head at a time,
    so that the scores of a long sequence fit."""
    tq, hq, _ = q.shape
    tk, hkv, _ = k.shape
    group = hq // hkv
    q_pos = torch.arange(tq, device=q.device) + (tk - tq)
    k_pos = torch.arange(tk, device=q.device)
    hidden = k_pos[None, :] > q_pos[:, None]
    if window is not None:
        hidden |= k_pos[None, :] < (q_pos[:, None] - window + 1)
    out = torch.empty_like(q)
    for h in range(hq):
        scores = (q[:, h] @ k[:, h // group].T) * scale
        scores = scores.masked_fill(hidden, float("-inf"))
        scores = scores - scores.max(dim=-1, keepdim=True).values
        weights = torch.exp(scores)
        out[:, h] = (weights / weights.sum(dim=-1, keepdim=True)) @ v[:, h // group]
    return out


def attention_layer(x, w_q, w_k, w_v, w_o, cos, sin, num_heads, num_kv_heads, head_dim, window=None, store=_keep):
    """models/blocks/gqa.py:107-154, scale 1/sqrt(D) (cache/packed_attention.py:126-127)."""
    t = x.shape[0]
    q = store(apply_rope(store(x @ w_q.T).reshape(t, num_heads, head_dim), cos, sin))
    k = store(apply_rope(store(x @ w_k.T).reshape(t, num_kv_heads, head_dim), cos, sin))
    v = store(x @ w_v.T).reshape(t, num_kv_heads, head_dim)
    out = store(causal_attention(q, k, v, 1.0 / math.sqrt(head_dim), window))
    return store(out.reshape(t, num_heads * head_dim) @ w_o.T)


def llama_logits(cfg: dict, weights: dict, token_ids, *, rows=None, store=_keep, device="cpu") -> np.ndarray:
    """Logits of one whole sequence as float64 NumPy [T, V] (or [len(rows), V]).

    models/llama/llama.py:149-172, models/blocks/transformer_block.py:95-153.  `weights` holds
    NumPy arrays or torch tensors under the checkpoint's names; `store` as in `plain_llama`.
    """
    def w(name: str) -> torch.Tensor:
        value = weights[name]
        if isinstance(value, np.ndarray):
            value = torch.from_numpy(value)
        return value.to(device=device, dtype=ACC)

    heads, kv_heads = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    head_dim = cfg.get("head_dim") or cfg["hidden_size"] // heads
    eps = cfg["rms_norm_eps"]
    ids = torch.as_tensor(np.asarray(token_ids, dtype=np.int64), device=device)
    inv_freq = torch.from_numpy(plain_llama.config_inv_freq(cfg)).to(device)
    cos, sin = rope_tables(torch.arange(len(ids), device=device), inv_freq)
    r = w("model.embed_tokens.weight")[ids]
    for layer in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{layer}."
        h = store(rms_norm(r, w(p + "input_layernorm.weight"), eps))
        r = r + attention_layer(
            h, w(p + "self_attn.q_proj.weight"), w(p + "self_attn.k_proj.weight"), w(p + "self_attn.v_proj.weight"),
            w(p + "self_attn.o_proj.weight"), cos, sin, heads, kv_heads, head_dim, store=store,
        )
        h = store(rms_norm(r, w(p + "post_attention_layernorm.weight"), eps))
        r = r + swiglu(h, w(p + "mlp.gate_proj.weight"), w(p + "mlp.up_proj.weight"), w(p + "mlp.down_proj.weight"), store)
    if rows is not None:
        r = r[torch.as_tensor(np.asarray(rows, dtype=np.int64), device=device)]
    h = store(rms_norm(r, w("model.norm.weight"), eps))
    head = "model.embed_tokens.weight" if cfg.get("tie_word_embeddings", False) else "lm_head.weight"
    return store(h @ w(head).T).cpu().numpy()
