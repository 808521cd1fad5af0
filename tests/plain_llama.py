"""A plain, slow NumPy implementation of the Llama decoder: whole sequences, no cache.

One function per part, written from the formulas of the reference
(JonathanBerhe/mini-infer; paths below are relative to its `src/mini_infer/`).
It shares no code with the engine.  Matrix products, norm statistics and the
softmax accumulate in float64 (`ACC`); the rotation angles follow the
reference's float32 arithmetic so both sides see the same table.

Weights are a dict of NumPy arrays under the checkpoint's tensor names.

`store` (optional, on the whole-model function and the parts it calls): a function
applied to every tensor that an engine computing in a narrower type would store in that
type (the output of each norm, projection, rotation, attention, activation and the
logits), with all arithmetic between still exact.  With `store=bf16_round` the model
shows how far bfloat16 storage alone moves the logits of a given input, which is the
yardstick the bfloat16 tests measure the engine's error with.  The residual stream is
not rounded (the engine keeps it in float32).
"""

from __future__ import annotations

import math

import numpy as np

ACC = np.float64


# ----------------------------------------------------------------------------
# position encoding
# ----------------------------------------------------------------------------


def inv_freq_default(head_dim: int, theta: float) -> np.ndarray:
    """`1 / theta^(2j/D)`, j = 0..D/2-1, in float32.

    models/blocks/rope.py:343-346 (`1.0 / base ** (arange(0, D, 2, dtype=float32) / D)`).
    The table is a float32 constant of the model, like a weight: an entry that differs in
    its last bit turns every key 2,000 positions away by another 1e-4 radians.  The
    reference makes it with torch's float32 power, whose last bits are not NumPy's (13 of
    the 64 entries differ for head size 128, theta 5e5), so this one line uses torch too.
    """
    import torch

    exponent = torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim
    return (1.0 / (theta**exponent)).numpy().astype(np.float32)


def inv_freq_llama3(
    inv_freq: np.ndarray,
    factor: float,
    low_freq_factor: float,
    high_freq_factor: float,
    original_max_position_embeddings: int,
) -> np.ndarray:
    """The llama3 rescale of an inverse-frequency table, float32 in and out.

    models/blocks/rope.py:200-225: wavelengths above L/low are divided by
    `factor`, those below L/high are kept, the band between is blended with
    `smooth = (L/wavelen - low) / (high - low)`.  Evaluated with torch's float32
    operations like the table itself (a Python number divided by a float32 tensor is
    rounded twice there, which moves last bits of the blended entries).
    """
    import torch

    table = torch.from_numpy(np.ascontiguousarray(inv_freq, dtype=np.float32))
    old_len = original_max_position_embeddings
    low_wavelen = old_len / low_freq_factor
    high_wavelen = old_len / high_freq_factor
    wavelen = 2 * math.pi / table
    scaled = torch.where(wavelen > low_wavelen, table / factor, table)
    smooth = (old_len / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
    smoothed = (1 - smooth) * scaled / factor + smooth * scaled
    medium = ~(wavelen < high_wavelen) & ~(wavelen > low_wavelen)
    return torch.where(medium, smoothed, scaled).numpy().astype(np.float32)


def rope_tables(positions: np.ndarray, inv_freq: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """`cos, sin` of shape [T, D]: angle = pos * inv_freq in float32, halves repeated.

    models/blocks/rope.py:392-408 (`freqs = inv_freq @ pos`, `emb = cat(freqs, freqs)`).
    """
    pos = positions.astype(np.float32)
    freqs = (pos[:, None] * inv_freq.astype(np.float32)[None, :]).astype(np.float32)
    emb = np.concatenate([freqs, freqs], axis=-1)
    return np.cos(emb.astype(ACC)), np.sin(emb.astype(ACC))


def rotate_half(x: np.ndarray) -> np.ndarray:
    """`(-x_high, x_low)` on the last axis.  models/blocks/rope.py:411-416."""
    half = x.shape[-1] // 2
    return np.concatenate([-x[..., half:], x[..., :half]], axis=-1)


def apply_rope(x: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
    """`x*cos + rotate_half(x)*sin` for x of shape [T, heads, D], tables [T, D].

    models/blocks/rope.py:419-431.
    """
    return x * cos[:, None, :] + rotate_half(x) * sin[:, None, :]


# ----------------------------------------------------------------------------
# norm, feed-forward, embedding
# ----------------------------------------------------------------------------


def rms_norm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """`w * x * rsqrt(mean(x^2) + eps)` over the last axis.

    models/blocks/rmsnorm.py:81-93.
    """
    x = x.astype(ACC)
    variance = np.mean(x * x, axis=-1, keepdims=True)
    return weight.astype(ACC) * (x / np.sqrt(variance + eps))


def silu(x: np.ndarray) -> np.ndarray:
    """`x / (1 + exp(-x))`.  models/blocks/silu_mul_kernel.py:86-90."""
    return x / (1.0 + np.exp(-x))


def _keep(x: np.ndarray) -> np.ndarray:
    return x


def bf16_round(x: np.ndarray) -> np.ndarray:
    """Values rounded to the nearest bfloat16 (ties to even), as float64."""
    bits = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    rounded = (bits + np.uint32(0x7FFF) + ((bits >> np.uint32(16)) & np.uint32(1))) & np.uint32(0xFFFF0000)
    return rounded.view(np.float32).astype(ACC)


def swiglu(x: np.ndarray, w_gate: np.ndarray, w_up: np.ndarray, w_down: np.ndarray, store=_keep) -> np.ndarray:
    """`down(silu(gate(x)) * up(x))`, weights in [out, in] layout, no biases.

    models/blocks/swiglu.py:44-46, models/blocks/activations.py:36-45.
    """
    x = x.astype(ACC)
    gate = store(x @ w_gate.astype(ACC).T)
    up = store(x @ w_up.astype(ACC).T)
    return store(store(silu(gate) * up) @ w_down.astype(ACC).T)


def embedding(table: np.ndarray, ids: np.ndarray) -> np.ndarray:
    """Row lookup.  models/llama/llama.py:159."""
    return table[ids].astype(ACC)


# ----------------------------------------------------------------------------
# attention
# ----------------------------------------------------------------------------


def causal_attention(
    q: np.ndarray,
    k: np.ndarray,
    v: np.ndarray,
    scale: float,
    window: int | None = None,
) -> np.ndarray:
    """Causal grouped-query attention of one whole sequence.

    q: [Tq, Hq, D]; k, v: [Tk, Hkv, D] with Tq <= Tk; the queries are the last
    Tq positions.  Query head h reads key/value head h // (Hq/Hkv); query at
    absolute position p sees keys 0..p, or p-window+1..p with a window.
    cache/packed_attention.py:296-338.
    """
    tq, hq, _ = q.shape
    tk, hkv, _ = k.shape
    if hq % hkv != 0:
        raise ValueError(f"num_q_heads={hq} not a multiple of num_kv_heads={hkv}")
    if tq > tk:
        raise ValueError(f"q_len={tq} > k_len={tk}")
    group = hq // hkv
    k = np.repeat(k.astype(ACC), group, axis=1)
    v = np.repeat(v.astype(ACC), group, axis=1)
    scores = np.einsum("qhd,khd->qhk", q.astype(ACC), k) * scale
    q_pos = np.arange(tq) + (tk - tq)
    k_pos = np.arange(tk)
    invalid = k_pos[None, :] > q_pos[:, None]
    if window is not None:
        invalid |= k_pos[None, :] < (q_pos[:, None] - window + 1)
    scores = np.where(invalid[:, None, :], -np.inf, scores)
    scores = scores - scores.max(axis=-1, keepdims=True)
    weights = np.exp(scores)
    weights = weights / weights.sum(axis=-1, keepdims=True)
    return np.einsum("qhk,khd->qhd", weights, v)


def attention_layer(
    x: np.ndarray,
    w_q: np.ndarray,
    w_k: np.ndarray,
    w_v: np.ndarray,
    w_o: np.ndarray,
    cos: np.ndarray,
    sin: np.ndarray,
    num_heads: int,
    num_kv_heads: int,
    head_dim: int,
    window: int | None = None,
    kv_override: tuple[np.ndarray, np.ndarray] | None = None,
    store=_keep,
) -> tuple[np.ndarray, tuple[np.ndarray, np.ndarray]]:
    """Project, rotate q and k, attend with scale 1/sqrt(D), project out.

    models/blocks/gqa.py:107-154 (scale: cache/packed_attention.py:126-127).
    Returns the output and the (rotated k, v) it used; `kv_override` makes the
    layer attend over another layer's keys and values instead of its own.
    """
    t = x.shape[0]
    x = x.astype(ACC)
    q = store(x @ w_q.astype(ACC).T).reshape(t, num_heads, head_dim)
    q = store(apply_rope(q, cos, sin))
    if kv_override is None:
        k = store(x @ w_k.astype(ACC).T).reshape(t, num_kv_heads, head_dim)
        v = store(x @ w_v.astype(ACC).T).reshape(t, num_kv_heads, head_dim)
        k = store(apply_rope(k, cos, sin))
    else:
        k, v = kv_override
    out = store(causal_attention(q, k, v, 1.0 / math.sqrt(head_dim), window))
    return store(out.reshape(t, num_heads * head_dim) @ w_o.astype(ACC).T), (k, v)


# ----------------------------------------------------------------------------
# whole model
# ----------------------------------------------------------------------------


def config_inv_freq(cfg: dict) -> np.ndarray:
    """The inverse-frequency table a config.json asks for.

    models/blocks/rope.py:228-269: `rope_parameters` or `rope_scaling`, type
    under `rope_type` or `type`, theta inside the dict or at top level.
    """
    head_dim = cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_attention_heads"]
    params = dict(cfg.get("rope_parameters") or cfg.get("rope_scaling") or {})
    theta = float(params.get("rope_theta") or cfg.get("rope_theta") or 10000.0)
    table = inv_freq_default(head_dim, theta)
    kind = params.get("rope_type") or params.get("type") or "default"
    if kind == "llama3":
        table = inv_freq_llama3(
            table,
            float(params["factor"]),
            float(params["low_freq_factor"]),
            float(params["high_freq_factor"]),
            int(params["original_max_position_embeddings"]),
        )
    elif kind != "default":
        raise NotImplementedError(kind)
    return table


def llama_logits(
    cfg: dict,
    weights: dict[str, np.ndarray],
    token_ids: np.ndarray,
    *,
    first_position: int = 0,
    order: list[tuple[int, int | None]] | None = None,
    window: int | None | list[int | None] = None,
    rows=None,
    store=_keep,
) -> np.ndarray:
    """Logits [T, V] of one whole sequence, float64 (with `rows`: of those positions only).

    models/llama/llama.py:149-172 and models/blocks/transformer_block.py:95-153:
    embed; per layer `r += attn(norm(r))`, `r += mlp(norm(r))`; final norm; head
    (the embedding table when `tie_word_embeddings`).

    `order` lists (layer, call whose keys and values it reads or None) in
    running order; the default runs every layer once with its own keys.
    `first_position` shifts all positions (only distances matter to the result).
    `window` is one window for every call, or a list with one entry per call.
    """
    heads = cfg["num_attention_heads"]
    kv_heads = cfg["num_key_value_heads"]
    head_dim = cfg.get("head_dim") or cfg["hidden_size"] // heads
    eps = cfg["rms_norm_eps"]
    ids = np.asarray(token_ids, dtype=np.int64)
    positions = np.arange(len(ids)) + first_position
    cos, sin = rope_tables(positions, config_inv_freq(cfg))

    if order is None:
        order = [(i, None) for i in range(cfg["num_hidden_layers"])]
    r = embedding(weights["model.embed_tokens.weight"], ids)
    kept: list[tuple[np.ndarray, np.ndarray]] = []
    windows = window if isinstance(window, list) else [window] * len(order)
    for call, (layer, reads) in enumerate(order):
        p = f"model.layers.{layer}."
        h = store(rms_norm(r, weights[p + "input_layernorm.weight"], eps))
        a, kv = attention_layer(
            h,
            weights[p + "self_attn.q_proj.weight"],
            weights[p + "self_attn.k_proj.weight"],
            weights[p + "self_attn.v_proj.weight"],
            weights[p + "self_attn.o_proj.weight"],
            cos,
            sin,
            heads,
            kv_heads,
            head_dim,
            windows[call],
            kv_override=None if reads is None else kept[reads],
            store=store,
        )
        kept.append(kv)
        r = r + a
        h = store(rms_norm(r, weights[p + "post_attention_layernorm.weight"], eps))
        r = r + swiglu(
            h,
            weights[p + "mlp.gate_proj.weight"],
            weights[p + "mlp.up_proj.weight"],
            weights[p + "mlp.down_proj.weight"],
            store=store,
        )
    if rows is not None:
        r = r[np.asarray(rows, dtype=np.int64)]
    h = store(rms_norm(r, weights["model.norm.weight"], eps))
    head = (
        weights["model.embed_tokens.weight"]
        if cfg.get("tie_word_embeddings", False)
        else weights["lm_head.weight"]
    )
    return store(h @ head.astype(ACC).T)


# ----------------------------------------------------------------------------
# sampling
# ----------------------------------------------------------------------------


def greedy(logits: np.ndarray) -> int:
    """First index of the maximum.  engine/sampler.py:26-27."""
    return int(np.argmax(logits))


def top_k_filter(logits: np.ndarray, k: int) -> np.ndarray:
    """Logits below the k-th largest become -inf; k = 0 or k >= V keeps all.

    engine/sampler.py:93-98.
    """
    if k <= 0 or k >= logits.shape[-1]:
        return logits
    threshold = np.sort(logits)[-k]
    return np.where(logits < threshold, -np.inf, logits)


def top_p_filter(logits: np.ndarray, p: float) -> np.ndarray:
    """Drop a token when the probability mass sorted before it exceeds p.

    engine/sampler.py:101-110 (the boundary token is kept).
    """
    if p >= 1.0:
        return logits
    order = np.argsort(-logits, kind="stable")
    sorted_logits = logits[order]
    probs = softmax(sorted_logits)
    cum = np.cumsum(probs)
    exclude = np.concatenate([[False], (cum > p)[:-1]])
    out = logits.copy()
    out[order[exclude]] = -np.inf
    return out


def softmax(x: np.ndarray) -> np.ndarray:
    x = x.astype(ACC)
    e = np.exp(x - np.max(x))
    return e / e.sum()


def sampling_distribution(
    logits: np.ndarray, temperature: float, top_k: int = 0, top_p: float = 1.0
) -> np.ndarray:
    """The distribution a sampling row draws from.  engine/sampler.py:29-35."""
    scaled = logits.astype(ACC) / temperature
    scaled = top_k_filter(scaled, top_k)
    scaled = top_p_filter(scaled, top_p)
    return softmax(scaled)
