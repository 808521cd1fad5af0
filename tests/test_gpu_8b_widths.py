"""One layer at the widths of Llama 3.1 8B (hidden 4096, 32/8 heads of 128, feed-forward
14336, llama3 rope) against the plain model: the sums over 4,096 and 14,336 terms, the
matrix-core attention at head size 128 and the weight-streaming GEMM shapes of the real
model, which the tiny configurations do not reach.  The vocabulary is cut to 32,077 to
keep the test short."""

import numpy as np
import pytest

import plain_llama
import replay_util as ru
import tiny

pytestmark = pytest.mark.gpu

WIDE = {
    "architectures": ["LlamaForCausalLM"],
    "num_hidden_layers": 1,
    "hidden_size": 4096,
    "num_attention_heads": 32,
    "num_key_value_heads": 8,
    "head_dim": 128,
    "intermediate_size": 14336,
    "vocab_size": 32077,
    "rope_theta": 500000.0,
    "rope_scaling": {
        "rope_type": "llama3",
        "factor": 8.0,
        "low_freq_factor": 1.0,
        "high_freq_factor": 4.0,
        "original_max_position_embeddings": 8192,
    },
    "rms_norm_eps": 1e-5,
    "tie_word_embeddings": False,
    "max_position_embeddings": 131072,
}


@pytest.fixture(scope="module")
def wide(tmp_path_factory):
    weights = tiny.make_weights(WIDE, seed=8)
    folder = tiny.write_model_dir(tmp_path_factory.mktemp("wide"), WIDE, weights)
    requests = {"p": tiny.random_tokens(WIDE, 45, seed=1), "q": tiny.random_tokens(WIDE, 23, seed=2)}
    expected = {rid: plain_llama.llama_logits(WIDE, weights, np.array(t)) for rid, t in requests.items()}
    return folder, requests, expected


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_real_widths_under_three_schedules(wide, dtype):
    from mini_infer_amd.engine import ModelRunner

    folder, requests, expected = wide
    runner = ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=8, block_size=16)
    schedules = {
        "whole": ru.schedule_whole(requests),
        "prefill+decode": ru.schedule_prefill_then_decode(requests, tail=12),
        "mixed": ru.schedule_mixed(requests, seed=3, max_live=2, tail=10),
    }
    for name, schedule in schedules.items():
        got = ru.run_schedule(runner, requests, schedule)
        for rid in requests:
            ru.assert_close(got[rid], expected[rid], dtype, f"8B widths, {name}, request {rid}")
        runner.cache.check()
    assert runner.num_free_blocks() == 8


def test_single_tokens_over_a_longer_context_at_real_widths(wide, monkeypatch):
    """One request of 600 tokens, the last 10 one by one in bfloat16 through the replayed decode
    step: at these widths and this context a single token's attention is left in its key ranges
    and combined by the output projection, and the down product is summed up by the next norm
    from 5 rows on (the 7-token portion)."""
    import mini_infer_amd.ops as ops
    from mini_infer_amd.engine import ModelRunner, StepEntry
    from mini_infer_amd.ops import kernels

    calls = {"from_attention": 0, "partial_sums": 0}
    from_attention, partial_sums = ops.linear_from_attention, kernels.linear_partial_sums

    def count_from_attention(*args):
        calls["from_attention"] += 1
        return from_attention(*args)

    def count_partial_sums(*args):
        calls["partial_sums"] += 1
        return partial_sums(*args)

    monkeypatch.setattr(ops, "linear_from_attention", count_from_attention)
    monkeypatch.setattr(kernels, "linear_partial_sums", count_partial_sums)
    folder, _, _ = wide
    tokens = tiny.random_tokens(WIDE, 600, seed=5)
    expected = plain_llama.llama_logits(WIDE, tiny.make_weights(WIDE, seed=8), np.array(tokens))  # the fixture's weights
    runner = ModelRunner.from_pretrained(folder, dtype="bfloat16", num_blocks=40, block_size=16)
    got = [runner.step([StepEntry("r", tokens[:583], [582])]).cpu().numpy()]
    got.append(runner.step([StepEntry("r", tokens[583:590], list(range(7)))]).cpu().numpy())
    for at in range(590, 600):
        got.append(runner.step([StepEntry("r", tokens[at : at + 1], [0])]).cpu().numpy())
    seen = expected.copy()
    seen[582:600] = np.concatenate(got)
    ru.assert_close(seen, expected, "bfloat16", "8B widths, 600 tokens")
    assert calls["from_attention"] >= 1 and calls["partial_sums"] >= 1  # (a replayed step calls nothing)
    runner.free_request("r")
    assert runner.num_free_blocks() == 40
