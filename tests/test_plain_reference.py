"""What fixes the plain implementation beside the reference's text (no GPU).

Each check is a vector the reference's own tests hold, a special case that
reduces to a library routine, or an invariant, chosen so that a plausible
mistake (a wrong sign or pairing, a norm in the wrong place, an off-by-one in
the mask) fails it.
"""

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import plain_llama as pl
import tiny


# -- inverse frequencies ------------------------------------------------------


def test_default_inv_freq():
    table = pl.inv_freq_default(16, 10000.0)
    assert table.dtype == np.float32 and table.shape == (8,)
    assert table[0] == 1.0
    assert np.all(np.diff(table) < 0)
    assert np.allclose(table, 10000.0 ** (-np.arange(0, 16, 2) / 16), rtol=1e-6)


def test_llama3_bands_of_the_tiny_table():
    """head_dim 16, theta 1e4, original length 64: "one kept, two blended, five divided"
    (the reference's tests/unit/models/llama/test_llama_rope_scaling.py:4-6)."""
    base = pl.inv_freq_default(16, 10000.0)
    scaled = pl.inv_freq_llama3(base, 8.0, 1.0, 4.0, 64)
    ratio = scaled / base
    kept = np.isclose(ratio, 1.0)
    divided = np.isclose(ratio, 1 / 8.0)
    blended = ~kept & ~divided
    assert kept.tolist() == [True] + [False] * 7
    assert blended.tolist() == [False, True, True] + [False] * 5
    assert divided.tolist() == [False] * 3 + [True] * 5
    assert np.all((ratio[blended] > 1 / 8.0) & (ratio[blended] < 1.0))


@pytest.mark.parametrize(
    "head_dim,theta,factor,orig,kept,blended",
    [(32, 500000.0, 8.0, 64, 2, 1), (128, 500000.0, 8.0, 8192, 29, 6), (128, 500000.0, 32.0, 8192, 29, 6)],
)
def test_llama3_bands_of_other_tables(head_dim, theta, factor, orig, kept, blended):
    base = pl.inv_freq_default(head_dim, theta)
    ratio = pl.inv_freq_llama3(base, factor, 1.0, 4.0, orig) / base
    is_kept, is_div = np.isclose(ratio, 1.0), np.isclose(ratio, 1 / factor)
    assert is_kept.sum() == kept and (~is_kept & ~is_div).sum() == blended
    assert is_kept[:kept].all() and is_div[kept + blended :].all()
    # band edges from the formula itself: wavelength against L/high and L/low
    wavelen = 2 * math.pi / base.astype(np.float64)
    assert np.array_equal(is_kept, wavelen < orig / 4.0)
    assert np.array_equal(is_div, wavelen > orig / 1.0)


def test_llama3_hand_computed_table():
    """The eight frequencies of head_dim 16, theta 1e4, factor 8, low 1, high 4, original
    length 64, worked out by hand from the reference's formula text (models/blocks/rope.py:200-225),
    with a calculator, not by running any implementation:

      j  inv_freq = 1e4^(-j/8)  wavelen = 2*pi/inv_freq   band (L/high = 16, L/low = 64)
      0  1                      6.2832                     < 16: kept            -> 1
      1  10^-0.5 = 0.3162278    19.8692                    blend, smooth = (64/19.86918 - 1)/3 = 0.7403565
                                 -> (1 - 0.7403565) * 0.3162278/8 + 0.7403565 * 0.3162278 = 0.2443846
      2  0.1                    62.8319                    blend, smooth = (64/62.8319 - 1)/3 = 0.0061972
                                 -> 0.9938028 * 0.0125 + 0.0061972 * 0.1 = 0.01304226
      3  10^-1.5 = 0.03162278   198.692                    > 64: divided         -> 0.003952847
      4  0.01                                                                     -> 0.00125
      5..7                                                                        -> inv_freq / 8

    A blend with `low` and `high` swapped, `1 - smooth` on the wrong term, or the band
    edges taken on frequencies instead of wavelengths changes entries 1 and 2.
    """
    got = pl.inv_freq_llama3(pl.inv_freq_default(16, 10000.0), 8.0, 1.0, 4.0, 64)
    by_hand = [1.0, 0.2443846, 0.01304226, 0.003952847, 0.00125, 10**-2.5 / 8, 1e-3 / 8, 10**-3.5 / 8]
    assert np.allclose(got, by_hand, rtol=2e-6, atol=0)
    # the same from the engine's own table builder
    from mini_infer_amd.parts.position import default_inv_freq, llama3_inv_freq

    ours = llama3_inv_freq(default_inv_freq(16, 10000.0), 8.0, 1.0, 4.0, 64).numpy()
    assert np.allclose(ours, by_hand, rtol=2e-6, atol=0)


def test_llama3_hand_computed_entry_of_the_released_table():
    """Llama 3.1's own numbers (head_dim 128, theta 5e5, factor 8, low 1, high 4, L 8192), entry 32:
    inv_freq = 5e5^(-0.5) = 0.001414214, wavelen = 4442.88 (between 2048 and 8192: blended),
    smooth = (8192/4442.883 - 1)/3 = 0.2812826,
    -> 0.7187174 * 0.001414214/8 + 0.2812826 * 0.001414214 = 0.0005248462."""
    got = pl.inv_freq_llama3(pl.inv_freq_default(128, 500000.0), 8.0, 1.0, 4.0, 8192)
    assert math.isclose(got[32], 0.0005248462, rel_tol=3e-6)
    assert math.isclose(got[0], 1.0) and math.isclose(got[63], 500000.0 ** (-126 / 128) / 8, rel_tol=1e-6)


def test_llama3_factor_one_is_identity():
    base = pl.inv_freq_default(64, 500000.0)
    assert np.allclose(pl.inv_freq_llama3(base, 1.0, 1.0, 4.0, 64), base, rtol=1e-6)


def test_engine_tables_equal_plain_tables():
    from mini_infer_amd.parts.position import default_inv_freq, llama3_inv_freq

    for head_dim, theta in ((16, 10000.0), (32, 500000.0), (128, 500000.0), (48, 20000.0)):
        ours = default_inv_freq(head_dim, theta).numpy()
        plain = pl.inv_freq_default(head_dim, theta)
        assert np.array_equal(ours, plain)  # bit for bit: one last bit is 1e-4 radians at position 2,000
        ours3 = llama3_inv_freq(torch.from_numpy(plain), 8.0, 1.0, 4.0, 64).numpy()
        assert np.array_equal(ours3, pl.inv_freq_llama3(plain, 8.0, 1.0, 4.0, 64))


# -- rotation -----------------------------------------------------------------------


def _rand(*shape, seed=0):
    return np.random.default_rng(seed).standard_normal(shape)


def test_rope_position_zero_is_identity():
    cos, sin = pl.rope_tables(np.array([0]), pl.inv_freq_default(16, 10000.0))
    x = _rand(1, 3, 16)
    assert np.allclose(pl.apply_rope(x, cos, sin), x)


def test_rope_is_a_complex_rotation_of_pairs_j_and_j_plus_half():
    """Half-rotation pairing: (x_j, x_{j+D/2}) -> multiply by exp(i * pos * inv_freq_j).
    An interleaved pairing, or a flipped sign, fails this."""
    head_dim = 16
    inv_freq = pl.inv_freq_default(head_dim, 10000.0)
    positions = np.array([0, 1, 5, 37])
    cos, sin = pl.rope_tables(positions, inv_freq)
    x = _rand(4, 2, head_dim, seed=1)
    out = pl.apply_rope(x, cos, sin)
    z = x[..., : head_dim // 2] + 1j * x[..., head_dim // 2 :]
    angle = positions[:, None].astype(np.float32) * inv_freq[None, :]
    rotated = z * np.exp(1j * angle.astype(np.float64))[:, None, :]
    assert np.allclose(out[..., : head_dim // 2], rotated.real, atol=1e-12)
    assert np.allclose(out[..., head_dim // 2 :], rotated.imag, atol=1e-12)
    # the norm of each pair is kept
    assert np.allclose(np.abs(rotated), np.abs(z))


def test_rope_scores_depend_on_distance_only():
    inv_freq = pl.inv_freq_default(32, 500000.0)
    q, k = _rand(1, 1, 32, seed=2), _rand(1, 1, 32, seed=3)

    def score(pq, pk):
        cq, sq = pl.rope_tables(np.array([pq]), inv_freq)
        ck, sk = pl.rope_tables(np.array([pk]), inv_freq)
        return float(np.sum(pl.apply_rope(q, cq, sq) * pl.apply_rope(k, ck, sk)))

    assert math.isclose(score(9, 4), score(105, 100), rel_tol=1e-4, abs_tol=1e-4)
    assert not math.isclose(score(9, 4), score(9, 5), rel_tol=1e-3)


# -- norm, feed-forward -------------------------------------------------------------


def test_rms_norm_against_the_library_and_invariants():
    x = _rand(5, 96, seed=4) * 3.0
    w = np.random.default_rng(5).uniform(0.5, 1.5, 96)
    ours = pl.rms_norm(x, w, 1e-5)
    lib = F.rms_norm(torch.from_numpy(x), (96,), torch.from_numpy(w), 1e-5).numpy()
    assert np.allclose(ours, lib, atol=1e-12)
    unit = pl.rms_norm(x, np.ones(96), 1e-12)
    assert np.allclose(np.sqrt((unit**2).mean(-1)), 1.0)
    assert np.allclose(pl.rms_norm(10 * x, w, 1e-12), pl.rms_norm(x, w, 1e-12))  # scale-invariant as eps -> 0
    const = pl.rms_norm(np.full((1, 8), -2.0), np.ones(8), 1e-6)
    assert np.allclose(const, -1.0 / math.sqrt(1 + 1e-6 / 4.0))
    # the weight multiplies after normalizing (not inside the mean)
    assert not np.allclose(ours, pl.rms_norm(x * w, np.ones(96), 1e-5))


def test_swiglu_against_the_library():
    x = _rand(4, 24, seed=6)
    wg, wu, wd = _rand(40, 24, seed=7), _rand(40, 24, seed=8), _rand(24, 40, seed=9)
    xt = torch.from_numpy(x)
    lib = (F.silu(xt @ torch.from_numpy(wg).T) * (xt @ torch.from_numpy(wu).T)) @ torch.from_numpy(wd).T
    assert np.allclose(pl.swiglu(x, wg, wu, wd), lib.numpy(), atol=1e-12)
    assert np.all(pl.swiglu(np.zeros((1, 24)), wg, wu, wd) == 0)
    assert np.isfinite(pl.silu(np.array([-80.0, 80.0]))).all()
    # gate and up are not interchangeable
    assert not np.allclose(pl.swiglu(x, wg, wu, wd), pl.swiglu(x, wu, wg, wd))


# -- attention ---------------------------------------------------------------------


def test_attention_whole_prompt_is_library_sdpa():
    q, k, v = _rand(9, 6, 16, seed=10), _rand(9, 2, 16, seed=11), _rand(9, 2, 16, seed=12)
    ours = pl.causal_attention(q, k, v, 0.25)
    tq = torch.from_numpy(q).transpose(0, 1)
    tk = torch.from_numpy(k).repeat_interleave(3, dim=1).transpose(0, 1)
    tv = torch.from_numpy(v).repeat_interleave(3, dim=1).transpose(0, 1)
    lib = F.scaled_dot_product_attention(tq, tk, tv, is_causal=True, scale=0.25).transpose(0, 1)
    assert np.allclose(ours, lib.numpy(), atol=1e-12)


def test_attention_special_cases():
    q, k, v = _rand(1, 4, 16, seed=13), _rand(1, 2, 16, seed=14), _rand(1, 2, 16, seed=15)
    out = pl.causal_attention(q, k, v, 0.25)
    assert np.allclose(out, np.repeat(v, 2, axis=1))  # one token attends to itself only
    # query head h reads key/value head h // group (not h % kv_heads)
    q, k, v = _rand(5, 4, 16, seed=16), _rand(5, 2, 16, seed=17), _rand(5, 2, 16, seed=18)
    out = pl.causal_attention(q, k, v, 0.25)
    for h in range(4):
        alone = pl.causal_attention(q[:, h : h + 1], k[:, h // 2 : h // 2 + 1], v[:, h // 2 : h // 2 + 1], 0.25)
        assert np.allclose(out[:, h : h + 1], alone)


def test_attention_chunk_offset_and_causality():
    q, k, v = _rand(12, 2, 16, seed=19), _rand(12, 1, 16, seed=20), _rand(12, 1, 16, seed=21)
    whole = pl.causal_attention(q, k, v, 0.3)
    tail = pl.causal_attention(q[7:], k, v, 0.3)  # the last five queries of the same sequence
    assert np.allclose(tail, whole[7:])
    poisoned_k, poisoned_v = k.copy(), v.copy()
    poisoned_k[8:] += 1000.0
    poisoned_v[8:] -= 1000.0
    assert np.allclose(pl.causal_attention(q, poisoned_k, poisoned_v, 0.3)[:8], whole[:8])
    with pytest.raises(ValueError):
        pl.causal_attention(q, k[:5], v[:5], 0.3)
    with pytest.raises(ValueError):
        pl.causal_attention(_rand(2, 3, 16), _rand(2, 2, 16), _rand(2, 2, 16), 0.3)


def test_attention_window():
    q, k, v = _rand(10, 1, 16, seed=22), _rand(10, 1, 16, seed=23), _rand(10, 1, 16, seed=24)
    assert np.allclose(pl.causal_attention(q, k, v, 0.3, window=10), pl.causal_attention(q, k, v, 0.3))
    windowed = pl.causal_attention(q, k, v, 0.3, window=3)
    # query 9 sees keys 7, 8, 9 only
    alone = pl.causal_attention(q[9:], k[7:], v[7:], 0.3)
    assert np.allclose(windowed[9:], alone)
    assert np.allclose(pl.causal_attention(q, k, v, 0.3, window=1), v)


# -- whole model -------------------------------------------------------------------


def test_model_logits_do_not_change_when_all_positions_shift():
    cfg, _ = tiny.CONFIGS["A"]
    weights = tiny.make_weights(cfg, 30)
    tokens = np.array(tiny.random_tokens(cfg, 12, 1))
    base = pl.llama_logits(cfg, weights, tokens)
    assert np.allclose(pl.llama_logits(cfg, weights, tokens, first_position=5), base, atol=1e-4)
    assert base.shape == (12, cfg["vocab_size"])


def test_model_is_causal_and_tied_head_is_the_embedding():
    cfg, _ = tiny.CONFIGS["A"]
    weights = tiny.make_weights(cfg, 31)
    tokens = np.array(tiny.random_tokens(cfg, 10, 2))
    base = pl.llama_logits(cfg, weights, tokens)
    changed = tokens.copy()
    changed[7] = (changed[7] + 1) % cfg["vocab_size"]
    other = pl.llama_logits(cfg, weights, changed)
    assert np.allclose(other[:7], base[:7]) and not np.allclose(other[7:], base[7:])
    untied = dict(cfg, tie_word_embeddings=False)
    with pytest.raises(KeyError):
        pl.llama_logits(untied, weights, tokens)
    weights["lm_head.weight"] = weights["model.embed_tokens.weight"]
    assert np.allclose(pl.llama_logits(untied, weights, tokens), base)


def test_model_one_layer_against_a_textbook_decoder_in_torch():
    """One layer, as many key heads as query heads: a decoder written with torch's own
    rms_norm, scaled_dot_product_attention and silu must give the same logits."""
    cfg = dict(tiny.TINY_A, num_hidden_layers=1, num_key_value_heads=4, tie_word_embeddings=True)
    weights = {k: v.astype(np.float64) for k, v in tiny.make_weights(cfg, 32).items()}
    tokens = tiny.random_tokens(cfg, 9, 3)
    t = {k: torch.from_numpy(v) for k, v in weights.items()}
    x = t["model.embed_tokens.weight"][tokens]
    cos, sin = (torch.from_numpy(a) for a in pl.rope_tables(np.arange(9), pl.config_inv_freq(cfg)))

    def rot(u):  # u: [T, heads, D]
        half = u.shape[-1] // 2
        return u * cos[:, None] + torch.cat([-u[..., half:], u[..., :half]], -1) * sin[:, None]

    p = "model.layers.0."
    h = F.rms_norm(x, (64,), t[p + "input_layernorm.weight"], cfg["rms_norm_eps"])
    q = rot((h @ t[p + "self_attn.q_proj.weight"].T).view(9, 4, 16)).transpose(0, 1)
    k = rot((h @ t[p + "self_attn.k_proj.weight"].T).view(9, 4, 16)).transpose(0, 1)
    v = (h @ t[p + "self_attn.v_proj.weight"].T).view(9, 4, 16).transpose(0, 1)
    a = F.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(0, 1).reshape(9, 64)
    x = x + a @ t[p + "self_attn.o_proj.weight"].T
    h = F.rms_norm(x, (64,), t[p + "post_attention_layernorm.weight"], cfg["rms_norm_eps"])
    x = x + (F.silu(h @ t[p + "mlp.gate_proj.weight"].T) * (h @ t[p + "mlp.up_proj.weight"].T)) @ t[
        p + "mlp.down_proj.weight"].T
    logits = F.rms_norm(x, (64,), t["model.norm.weight"], cfg["rms_norm_eps"]) @ t["model.embed_tokens.weight"].T
    assert np.allclose(pl.llama_logits(cfg, weights, np.array(tokens)), logits.numpy(), atol=1e-9)


def test_order_list_and_cache_reading():
    cfg, _ = tiny.CONFIGS["A"]
    weights = tiny.make_weights(cfg, 33)
    tokens = np.array(tiny.random_tokens(cfg, 8, 4))
    base = pl.llama_logits(cfg, weights, tokens)
    assert np.allclose(pl.llama_logits(cfg, weights, tokens, order=[(0, None), (1, None)]), base)
    looped = pl.llama_logits(cfg, weights, tokens, order=[(0, None), (1, None), (0, None)])
    shared = pl.llama_logits(cfg, weights, tokens, order=[(0, None), (1, 0)])
    assert not np.allclose(looped, base) and not np.allclose(shared, base)


def test_torch_twin_of_the_plain_model_equals_it():
    """`plain_llama_torch` (the same formulas in torch float64, for inputs too large for NumPy) is
    pinned to the NumPy implementation on all tiny configurations, with and without rounding
    of the stored tensors, whole and at chosen rows."""
    import plain_llama_torch as plt

    for name in "ABCDEF":
        cfg, _ = tiny.CONFIGS[name]
        weights = tiny.make_weights(cfg, 40 + ord(name))
        tokens = tiny.random_tokens(cfg, 70, 5)
        exact = pl.llama_logits(cfg, weights, np.array(tokens))
        assert np.abs(plt.llama_logits(cfg, weights, tokens) - exact).max() < 1e-9
        assert np.abs(plt.llama_logits(cfg, weights, tokens, rows=[0, 41, 69]) - exact[[0, 41, 69]]).max() < 1e-9
        rounded = pl.llama_logits(cfg, weights, np.array(tokens), store=pl.bf16_round)
        twin = plt.llama_logits(cfg, weights, tokens, store=plt.bf16_round)
        # a value that sits on a rounding boundary may fall to either side in the two libraries
        assert np.mean(np.abs(twin - rounded) > 1e-9) < 0.02
        assert 0 < np.abs(rounded - exact).max() < 0.05 * np.abs(exact).max()


def test_bf16_round_is_round_to_nearest_even():
    x = np.array([1.0, 1.00390625, 1.01171875, -3.0e-40, 65280.0, 1.0 + 2.0**-9], dtype=np.float64)
    assert np.array_equal(pl.bf16_round(x), torch.from_numpy(x).float().bfloat16().double().numpy())
    assert pl.bf16_round(np.array([1.00390625]))[0] == 1.0  # a tie goes to the even neighbour
    assert pl.bf16_round(np.array([1.01171875]))[0] == 1.015625


# -- sampling ---------------------------------------------------------------------


def test_greedy_and_filters():
    logits = np.array([1.0, 5.0, 3.0, 5.0, 2.0])
    assert pl.greedy(logits) == 1  # ties: first index (tests/unit/engine/test_sampler.py:18-21 of the reference)
    assert np.array_equal(np.isfinite(pl.top_k_filter(logits, 2)), [False, True, False, True, False])
    assert np.array_equal(pl.top_k_filter(logits, 0), logits) and np.array_equal(pl.top_k_filter(logits, 9), logits)
    one = np.array([1.0, 5.0, 3.0, 2.0])
    assert np.array_equal(np.isfinite(pl.top_p_filter(one, 0.001)), [False, True, False, False])
    probs = pl.softmax(one)
    keep_two = probs[1] + probs[2] / 2  # the boundary token (index 2) stays
    assert np.array_equal(np.isfinite(pl.top_p_filter(one, keep_two)), [False, True, True, False])
    assert np.array_equal(pl.top_p_filter(one, 1.0), one)
    dist = pl.sampling_distribution(one, 2.0, top_k=3)
    assert dist[0] == 0 and math.isclose(dist.sum(), 1.0) and dist[1] > dist[2] > dist[3]
    assert np.allclose(pl.sampling_distribution(one, 1.0), probs)
