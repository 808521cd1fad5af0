"""Configurations drawn at random, each replayed whole and mixed against the plain model.

The tiny configurations of `tiny.py` are chosen by hand; these are not.  A seed fixes the
sizes (heads, groups, head sizes that are and are not multiples of 16, a width that need not be
heads x head size, odd feed-forward widths and vocabularies, depth, eps, rope base and scaling,
tied or untied head) and the weights; the model is then run whole and in the mixed schedule,
with so few pages that they are used again, in float32 and in bfloat16, at the engine's
default page size.  Wide seeds draw widths in multiples of 64 and head sizes of 64 to 128, at
which the bfloat16 engine takes its fast kernels (whole weight lines, norms folded into the
products, the matrix-core attention).
"""

import numpy as np
import pytest

import replay_util as ru
import tiny

pytestmark = pytest.mark.gpu

PAGE = 16


def random_config(seed: int, wide: bool) -> dict:
    rng = np.random.default_rng(seed)
    kv_heads = int(rng.integers(1, 5))
    heads = kv_heads * int(rng.choice([1, 2, 3, 4, 5, 7, 8]))
    if wide:
        head_dim = int(rng.choice([64, 128, 96, 80]))
        hidden = 64 * int(rng.integers(2, 25))
        intermediate = int(rng.choice([64, 128, 32])) * int(rng.integers(3, 40))
        vocab = int(rng.integers(500, 9000))
        layers = int(rng.integers(1, 4))
    else:
        head_dim = int(rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 24, 40, 100, 18, 160, 256]))
        hidden = int(rng.choice([int(rng.integers(16, 400)) * 2, heads * head_dim, int(rng.integers(33, 500))]))
        intermediate = int(rng.choice([int(rng.integers(8, 700)), int(rng.integers(4, 300)) * 2]))
        vocab = int(rng.integers(40, 3000))
        layers = int(rng.integers(1, 5))
    cfg = {
        "architectures": ["LlamaForCausalLM"],
        "num_hidden_layers": layers,
        "hidden_size": hidden,
        "num_attention_heads": heads,
        "num_key_value_heads": kv_heads,
        "head_dim": head_dim,
        "intermediate_size": intermediate,
        "vocab_size": vocab,
        "rope_theta": float(rng.choice([10000.0, 500000.0, 1000000.0, 777.0])),
        "rms_norm_eps": float(rng.choice([1e-5, 1e-6, 3e-4])),
        "tie_word_embeddings": bool(rng.integers(0, 2)),
        "max_position_embeddings": 4096,
    }
    if hidden == heads * head_dim and rng.integers(0, 2):
        del cfg["head_dim"]  # then it is hidden_size / num_attention_heads
    if rng.integers(0, 2):
        cfg["rope_scaling"] = {
            "rope_type": "llama3",
            "factor": float(rng.choice([2.0, 8.0, 32.0])),
            "low_freq_factor": 1.0,
            "high_freq_factor": float(rng.choice([2.0, 4.0])),
            "original_max_position_embeddings": int(rng.choice([16, 64, 8192])),
        }
    return cfg


def _weights(cfg: dict, seed: int) -> dict:
    """`tiny.make_weights`, with a tied table scaled down so that the logits stay of order ten
    at every width (the float32 bound is absolute, and float32 itself is relative)."""
    weights = tiny.make_weights(cfg, seed)
    if cfg["tie_word_embeddings"]:
        table = weights["model.embed_tokens.weight"] * (4.0 / np.sqrt(cfg["hidden_size"]))
        weights["model.embed_tokens.weight"] = tiny.bf16_round(table.astype(np.float32))
    return weights


SEEDS = [(seed, False) for seed in range(1000, 1008)] + [(seed, True) for seed in range(2000, 2006)]


@pytest.fixture(scope="module", params=SEEDS, ids=lambda p: f"{'wide' if p[1] else 'any'}{p[0]}")
def case(request, tmp_path_factory):
    seed, wide = request.param
    cfg = random_config(seed, wide)
    weights = _weights(cfg, seed)
    folder = tiny.write_model_dir(tmp_path_factory.mktemp(f"random{seed}"), cfg, weights)
    rng = np.random.default_rng(seed + 1)
    lengths = [int(rng.integers(40, 200)) for _ in range(5)]
    requests = {f"r{i}": tiny.random_tokens(cfg, n, seed=seed * 10 + i) for i, n in enumerate(lengths)}
    expected = {rid: ru.oracle(cfg, weights, t) for rid, t in requests.items()}
    return seed, cfg, folder, requests, expected


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_random_configuration_whole_and_mixed_with_page_reuse(case, dtype):
    from mini_infer_amd.engine import ModelRunner

    seed, cfg, folder, requests, expected = case
    print(f"seed {seed}: {cfg}", flush=True)
    for what, schedule in (("whole", ru.schedule_whole(requests)), ("mixed", ru.schedule_mixed(requests, seed=seed))):
        pages = ru.peak_pages(requests, schedule, PAGE)
        runner = ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=pages, block_size=PAGE)
        got = ru.run_schedule(runner, requests, schedule)
        for rid in requests:
            ru.assert_close(got[rid], expected[rid], dtype, f"seed {seed} {what} request {rid}")
        runner.cache.check()
        assert runner.num_free_blocks() == runner.num_blocks
