"""The engine against the plain model under every way of cutting the work.

For each tiny configuration, in float32 and in bfloat16: each request alone and
whole; most of it in one step and the last 32 tokens one by one; portions of
changing size down to two tokens; and mixed, up to four live requests with so
few pages that they are used again.  Logits at every position must agree with
the plain whole-sequence model.
"""

import numpy as np
import pytest

import replay_util as ru
import tiny

pytestmark = pytest.mark.gpu

LENGTHS = [5, 33, 70, 97, 41, 64]


@pytest.fixture(scope="module", params=["A", "B", "C", "D", "E", "F"])
def case(request, tmp_path_factory):
    name = request.param
    cfg, block = tiny.CONFIGS[name]
    weights = tiny.make_weights(cfg, seed=100 + ord(name))
    folder = tiny.write_model_dir(tmp_path_factory.mktemp(f"model{name}"), cfg, weights)
    requests = {f"r{i}": tiny.random_tokens(cfg, n, seed=i) for i, n in enumerate(LENGTHS)}
    expected = {rid: ru.oracle(cfg, weights, t) for rid, t in requests.items()}
    return name, cfg, block, folder, requests, expected


def _runner(folder, dtype, block, pages):
    from mini_infer_amd.engine import ModelRunner

    return ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=pages, block_size=block)


def _check(runner, requests, expected, schedule, dtype, what):
    got = ru.run_schedule(runner, requests, schedule)
    for rid in requests:
        ru.assert_close(got[rid], expected[rid], dtype, f"{what} request {rid}")
    runner.cache.check()
    assert runner.num_free_blocks() == runner.num_blocks, "pages were not all given back"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole(case, dtype):
    name, cfg, block, folder, requests, expected = case
    _check(_runner(folder, dtype, block, 64), requests, expected, ru.schedule_whole(requests), dtype, f"{name} whole")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prefill_then_decode(case, dtype, monkeypatch):
    import mini_infer_amd.ops as ops

    name, cfg, block, folder, requests, expected = case
    folded = {"products": 0, "scaled_rows": 0}
    add_norm, rope_write = ops.linear_add_norm, ops.qkv_rope_write

    def count_add_norm(*args):
        folded["products"] += 1
        return add_norm(*args)

    def count_rope_write(x, *args, **kwargs):
        folded["scaled_rows"] += isinstance(x, ops.ScaledRows)
        return rope_write(x, *args, **kwargs)

    monkeypatch.setattr(ops, "linear_add_norm", count_add_norm)
    monkeypatch.setattr(ops, "qkv_rope_write", count_rope_write)
    schedule = ru.schedule_prefill_then_decode(requests)
    _check(_runner(folder, dtype, block, 64), requests, expected, schedule, dtype, f"{name} prefill+decode")
    if name == "D" and dtype == "bfloat16":
        # the configuration whose sizes the folded kernels take: both norms of a layer went that way
        assert folded["products"] >= 2 * cfg["num_hidden_layers"] - 1 and folded["scaled_rows"] >= 1
    if dtype == "float32":
        assert folded == {"products": 0, "scaled_rows": 0}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions(case, dtype):
    name, cfg, block, folder, requests, expected = case
    schedule = ru.schedule_portions(requests, seed=3)
    assert any(c == 2 for s in schedule for c in s["feed"].values())
    _check(_runner(folder, dtype, block, 64), requests, expected, schedule, dtype, f"{name} portions")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_with_page_reuse(case, dtype):
    name, cfg, block, folder, requests, expected = case
    schedule = ru.schedule_mixed(requests, seed=11)
    assert max(len(s["feed"]) for s in schedule) == 4
    assert any(
        any(c > 1 for c in s["feed"].values()) and any(c == 1 for c in s["feed"].values()) for s in schedule
    ), "no step mixes a portion with a single token"
    pages = ru.peak_pages(requests, schedule, block)
    total_pages = sum(-(-len(t) // block) for t in requests.values())
    assert pages < total_pages, "the pool is not small enough to force reuse"
    _check(_runner(folder, dtype, block, pages), requests, expected, schedule, dtype, f"{name} mixed")
