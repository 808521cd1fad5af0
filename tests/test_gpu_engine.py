"""The engine above the kernels: parts alone, generation through the entry points,
the replay program, long decoding, first tokens, order lists, windows, and a toy
mixer with state of its own registered from outside the package."""

import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_llama as pl
import replay_util as ru
import tiny

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = ["float32", "bfloat16"]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def _folder(tmp_path, name, seed):
    cfg, block = tiny.CONFIGS[name]
    weights = tiny.make_weights(cfg, seed)
    return cfg, block, weights, tiny.write_model_dir(tmp_path / f"model{name}{seed}", cfg, weights)


def _plain_greedy(cfg, weights, prompt, count):
    sequence = list(prompt)
    for _ in range(count):
        sequence.append(pl.greedy(pl.llama_logits(cfg, weights, np.array(sequence))[-1]))
    return sequence[len(prompt):]


# -- parts alone -----------------------------------------------------------------


def _context(positions, cu, seq_lens, slot_mapping=None, block_table=None, page_size=4):
    from mini_infer_amd.parts import StepContext

    t = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)  # noqa: E731
    token_request = [b for b in range(len(cu) - 1) for _ in range(cu[b + 1] - cu[b])]
    return StepContext(
        num_tokens=len(positions), num_requests=len(cu) - 1, page_size=page_size, token_ids=t([0] * len(positions)),
        positions=t(positions), token_request=t(token_request), cu_seqlens_q=t(cu), seq_lens=t(seq_lens),
        state_slots=t(list(range(len(cu) - 1))), logit_rows=t([]),
        slot_mapping=[t(slot_mapping)] if slot_mapping is not None else [],
        block_tables=[t(block_table)] if block_table is not None else [],
        max_q_len=max(cu[b + 1] - cu[b] for b in range(len(cu) - 1)), max_seq_len=max(seq_lens),
        host_cu_seqlens_q=cu, host_seq_lens=seq_lens, host_state_slots=list(range(len(cu) - 1)))


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_part(dtype):
    from mini_infer_amd.registry import NORMS

    norm = NORMS.lookup("rms_norm")({"kind": "rms_norm", "hidden_size": 100, "eps": 2e-6}, TORCH[dtype], DEV)
    assert list(norm.param_specs("x.")) == ["x.weight"]
    w = torch.rand(100) + 0.5
    norm.load_params("x.", lambda name: w.to(TORCH[dtype]).to(DEV))
    residual = torch.randn(3, 100, device=DEV)
    delta = torch.randn(3, 100, device=DEV).to(TORCH[dtype])
    expected = pl.rms_norm((residual.double() + delta.double()).cpu().numpy(),
                           w.to(TORCH[dtype]).double().numpy(), 2e-6)
    out = norm.forward(delta, residual)
    assert np.abs(out.float().cpu().numpy() - expected).max() < (1e-5 if dtype == "float32" else 4e-2)


def test_position_part():
    """The rotary part alone, built through the registry: the llama3 rescale of the table and
    the angles in float32 as the plain model makes them, at positions up to the model's reach;
    one table per step, shared by every layer that asks."""
    from mini_infer_amd.registry import POSITION_ENCODINGS

    llama3 = {"factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}
    for desc, table in (
        ({"kind": "rotary", "head_dim": 128, "theta": 500000.0, "llama3": llama3},
         pl.inv_freq_llama3(pl.inv_freq_default(128, 500000.0), 8.0, 1.0, 4.0, 8192)),
        ({"kind": "rotary", "head_dim": 48, "theta": 100.0}, pl.inv_freq_default(48, 100.0)),
        ({"kind": "rotary", "head_dim": 48, "theta": 100.0, "rotary_dim": 16}, pl.inv_freq_default(16, 100.0)),
    ):
        part = POSITION_ENCODINGS.lookup("rotary")(desc, torch.bfloat16, DEV)
        assert part.param_specs("x.") == {}
        ours = part.inv_freq.cpu().numpy()
        assert ours.dtype == np.float32 and np.allclose(ours, table, rtol=5e-7, atol=0)  # an ulp or two of the power
        positions = [0, 1, 2, 8191, 8192, 131071, 5, 70000]
        ctx = _context(positions, [0, len(positions)], [131072])
        cos, sin = part.tables(ctx)
        assert cos.dtype == torch.float32 and cos.shape == (len(positions), len(table))
        want_cos, want_sin = pl.rope_tables(np.array(positions), ours)
        # the angle is one float32 product, here as there; cos and sin of it within float32 rounding
        assert np.abs(cos.cpu().numpy() - want_cos[:, : len(table)]).max() < 2e-6
        assert np.abs(sin.cpu().numpy() - want_sin[:, : len(table)]).max() < 2e-6
        assert part.tables(ctx)[0] is cos  # made once a step


@pytest.mark.parametrize("dtype", DTYPES)
def test_feed_forward_part(dtype):
    from mini_infer_amd.registry import FEED_FORWARDS

    ffn = FEED_FORWARDS.lookup("swiglu")(
        {"kind": "swiglu", "hidden_size": 90, "intermediate_size": 130}, TORCH[dtype], DEV)
    assert sorted(ffn.param_specs("m.")) == ["m.down_proj.weight", "m.gate_proj.weight", "m.up_proj.weight"]
    rng = np.random.default_rng(0)
    w = {"m.gate_proj.weight": rng.standard_normal((130, 90)) / 9, "m.up_proj.weight": rng.standard_normal((130, 90)) / 9,
         "m.down_proj.weight": rng.standard_normal((90, 130)) / 11}
    w = {k: tiny.bf16_round(v) for k, v in w.items()}
    ffn.load_params("m.", lambda name: torch.from_numpy(w[name]).to(TORCH[dtype]).to(DEV))
    x = torch.from_numpy(tiny.bf16_round(rng.standard_normal((5, 90)))).to(DEV)
    expected = pl.swiglu(x.cpu().numpy(), w["m.gate_proj.weight"], w["m.up_proj.weight"], w["m.down_proj.weight"])
    out = ffn.forward(x.to(TORCH[dtype]), None)
    assert np.abs(out.float().cpu().numpy() - expected).max() < (1e-5 if dtype == "float32" else 4e-2)
    with pytest.raises(NotImplementedError):
        FEED_FORWARDS.lookup("swiglu")({"kind": "swiglu", "hidden_size": 8, "intermediate_size": 8,
                                        "activation": "gelu"}, TORCH[dtype], DEV)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [None, 5])
def test_attention_part_in_two_portions(dtype, window):
    """The mixer alone: a sequence fed as 7 + 4 tokens through its own little cache."""
    from mini_infer_amd.parts import LayerCache
    from mini_infer_amd.registry import MIXERS

    hidden, heads, kv_heads, head_dim, page = 40, 6, 2, 16, 4
    desc = {"kind": "gqa_attention", "hidden_size": hidden, "num_heads": heads, "num_kv_heads": kv_heads,
            "head_dim": head_dim, "window": window,
            "position": {"kind": "rotary", "head_dim": head_dim, "theta": 100.0}}
    mixer = MIXERS.lookup("gqa_attention")(desc, TORCH[dtype], DEV, {})
    needs = mixer.cache_needs(4)
    assert (needs.pages.num_kv_heads, needs.pages.head_dim, needs.pages.window) == (kv_heads, head_dim, window)
    rng = np.random.default_rng(1)
    w = {f"a.{n}_proj.weight": tiny.bf16_round(rng.standard_normal(s) / 6) for n, s in
         (("q", (96, 40)), ("k", (32, 40)), ("v", (32, 40)), ("o", (40, 96)))}
    mixer.load_params("a.", lambda name: torch.from_numpy(w[name]).to(TORCH[dtype]).to(DEV))
    x = tiny.bf16_round(rng.standard_normal((11, hidden)))
    cos, sin = pl.rope_tables(np.arange(11), pl.inv_freq_default(head_dim, 100.0))
    expected, _ = pl.attention_layer(x, w["a.q_proj.weight"], w["a.k_proj.weight"], w["a.v_proj.weight"],
                                     w["a.o_proj.weight"], cos, sin, heads, kv_heads, head_dim, window)
    cache = LayerCache(group=0, k_pages=torch.zeros((5, kv_heads, page, head_dim), dtype=TORCH[dtype], device=DEV),
                       v_pages=torch.zeros((5, kv_heads, page, head_dim), dtype=TORCH[dtype], device=DEV))
    table = [[3, 0, 4]]
    slots = [table[0][p // page] * page + p % page for p in range(11)]
    xt = torch.from_numpy(x).to(TORCH[dtype]).to(DEV)
    first = mixer.forward(xt[:7], _context(list(range(7)), [0, 7], [7], slots[:7], table), cache)
    second = mixer.forward(xt[7:], _context(list(range(7, 11)), [0, 4], [11], slots[7:], table), cache)
    got = torch.cat([first, second]).float().cpu().numpy()
    assert np.abs(got - expected).max() < (2e-5 if dtype == "float32" else 4e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_block_part_arranges_norms_mixer_and_feed_forward_around_the_residual(dtype):
    """The pre-norm block alone, built through the registry: what comes in still to be added
    is added by its first norm, the mixer's output by its second, and its own feed-forward
    output goes out unadded (models/blocks/transformer_block.py:95-120)."""
    from mini_infer_amd.parts import LayerCache
    from mini_infer_amd.registry import BLOCKS

    hidden, heads, kv_heads, head_dim, inter, page, eps, n = 40, 6, 2, 16, 56, 4, 3e-6, 9
    desc = {
        "kind": "pre_norm",
        "norm": {"kind": "rms_norm", "hidden_size": hidden, "eps": eps},
        "mixer": {"kind": "gqa_attention", "hidden_size": hidden, "num_heads": heads, "num_kv_heads": kv_heads,
                  "head_dim": head_dim, "window": None,
                  "position": {"kind": "rotary", "head_dim": head_dim, "theta": 100.0}},
        "feed_forward": {"kind": "swiglu", "hidden_size": hidden, "intermediate_size": inter},
        "names": {"mixer_norm": "n1.", "mixer": "att.", "ffn_norm": "n2.", "feed_forward": "ff."},
    }
    block = BLOCKS.lookup("pre_norm")(desc, TORCH[dtype], DEV, {})
    rng = np.random.default_rng(4)
    shapes = {"n1.weight": (hidden,), "n2.weight": (hidden,), "att.q_proj.weight": (heads * head_dim, hidden),
              "att.k_proj.weight": (kv_heads * head_dim, hidden), "att.v_proj.weight": (kv_heads * head_dim, hidden),
              "att.o_proj.weight": (hidden, heads * head_dim), "ff.gate_proj.weight": (inter, hidden),
              "ff.up_proj.weight": (inter, hidden), "ff.down_proj.weight": (hidden, inter)}
    assert set(block.param_specs("L.")) == {"L." + name for name in shapes}
    w = {name: tiny.bf16_round(1 + rng.standard_normal(s) / 10 if len(s) == 1 else rng.standard_normal(s) / 6)
         for name, s in shapes.items()}
    block.load_params("L.", lambda name: torch.from_numpy(w[name[2:]]).to(TORCH[dtype]).to(DEV))
    x = tiny.bf16_round(rng.standard_normal((n, hidden)))
    incoming = tiny.bf16_round(rng.standard_normal((n, hidden)))
    # plain: the residual takes the incoming piece, then the mixer's; the feed-forward's stays apart
    cos, sin = pl.rope_tables(np.arange(n), pl.inv_freq_default(head_dim, 100.0))
    stream = x + incoming
    mixed, _ = pl.attention_layer(pl.rms_norm(stream, w["n1.weight"], eps), w["att.q_proj.weight"],
                                  w["att.k_proj.weight"], w["att.v_proj.weight"], w["att.o_proj.weight"], cos, sin,
                                  heads, kv_heads, head_dim, None)
    stream = stream + mixed
    out = pl.swiglu(pl.rms_norm(stream, w["n2.weight"], eps), w["ff.gate_proj.weight"], w["ff.up_proj.weight"],
                    w["ff.down_proj.weight"])
    cache = LayerCache(group=0, k_pages=torch.zeros((4, kv_heads, page, head_dim), dtype=TORCH[dtype], device=DEV),
                       v_pages=torch.zeros((4, kv_heads, page, head_dim), dtype=TORCH[dtype], device=DEV))
    table = [[2, 0, 3]]
    slots = [table[0][p // page] * page + p % page for p in range(n)]
    residual = torch.from_numpy(x).float().to(DEV)
    delta = torch.from_numpy(incoming).to(TORCH[dtype]).to(DEV)
    got = block.forward(delta, residual, _context(list(range(n)), [0, n], [n], slots, table), cache)
    tol = 3e-5 if dtype == "float32" else 6e-2
    assert np.abs(residual.cpu().numpy() - stream).max() < tol
    assert np.abs(got.float().cpu().numpy() - out).max() < tol


# -- generation through the entry points ---------------------------------------------


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_llm(tmp_path, name):
    """Tiny A: 3 requests (5, 17, 32 tokens), 8 greedy tokens each, block size 4.
    Tiny B: 4 requests (1, 40, 97, 150 tokens) under a 32-token budget, block size 16."""
    from mini_infer_amd.engine.llm import LLM

    cfg, block, weights, folder = _folder(tmp_path, name, 50)
    lengths, new_tokens = ((5, 17, 32), 8) if name == "A" else ((1, 40, 97, 150), 12)
    prompts = [tiny.random_tokens(cfg, n, seed=n) for n in lengths]
    llm = LLM(folder, dtype="float32", num_blocks=96, block_size=block, max_num_batched_tokens=32, chunk_size=32)
    results = llm.generate(prompts, max_tokens=new_tokens)
    for prompt, result in zip(prompts, results):
        assert result.tokens == _plain_greedy(cfg, weights, prompt, new_tokens)
        assert result.finish_reason == "length" and result.prompt_tokens == len(prompt)
    assert llm.runner.num_free_blocks() == 96
    stats = llm.scheduler.stats
    # every prompt token and every generated token but each request's last went through the model once
    assert stats["tokens_run"] == sum(lengths) + len(lengths) * (new_tokens - 1)
    assert stats["preemptions"] == 0 and stats["rejected"] == 0
    # The steps, counted by hand from the policy (decoding requests first, then portions in
    # admission order under the 32-token budget; a request's first token comes from the step that
    # ends its prompt, its n-th from n - 1 steps later).  A: 5 + 17 + 10 | 2 + 22 | then single
    # tokens: the last prompt ends in step 1, so its 8th token comes from step 8: 9 steps.
    # B: 1 + 31 | 1 + 9 + 22 | 2 + 30 | 2 + 30 | 2 + 15 + 15 | 3 + 29 (four times) | 3 + 19: the
    # last prompt ends in step 9, its 12th token comes from step 20: 21 steps.
    assert stats["steps"] == (9 if name == "A" else 21)


def test_greedy_generation_in_bfloat16_stays_on_near_maxima(tmp_path):
    """bfloat16 may pick another token where two logits nearly tie; every token it picks
    must be within rounding of the plain model's maximum given the engine's own prefix."""
    from mini_infer_amd.engine.llm import LLM

    cfg, block, weights, folder = _folder(tmp_path, "B", 51)
    prompts = [tiny.random_tokens(cfg, n, seed=n) for n in (3, 40)]
    llm = LLM(folder, dtype="bfloat16", num_blocks=32, block_size=block)
    for prompt, result in zip(prompts, llm.generate(prompts, max_tokens=10)):
        sequence = list(prompt)
        for token in result.tokens:
            plain = ru.oracle(cfg, weights, sequence)
            logits = plain.exact[-1]
            # both the chosen logit and the largest one may be off by the bound of `assert_close`
            assert logits[token] > logits.max() - 2 * ru.BF16_MAX_FACTOR * plain.yard_max
            sequence.append(token)


def test_seeded_temperature_generation_is_reproducible_and_independent_of_batching(tmp_path):
    """Two greedy and two sampled requests (temperature 0.8): the sampled ones give the
    same tokens alone, batched, and under another chunking."""
    from mini_infer_amd.engine.llm import LLM
    from mini_infer_amd.sampling import SamplingParams

    cfg, block, weights, folder = _folder(tmp_path, "B", 52)
    prompts = [tiny.random_tokens(cfg, n, seed=n) for n in (1, 40, 97, 150)]
    params = [SamplingParams(), SamplingParams(temperature=0.8, seed=7), SamplingParams(),
              SamplingParams(temperature=0.8, seed=8, top_k=50, top_p=0.9)]
    batched = LLM(folder, dtype="float32", num_blocks=96, block_size=block, max_num_batched_tokens=32,
                  chunk_size=32).generate(prompts, params, max_tokens=12)
    other = LLM(folder, dtype="float32", num_blocks=96, block_size=block, max_num_batched_tokens=512,
                max_concurrent=2).generate(prompts, params, max_tokens=12)
    assert [r.tokens for r in batched] == [r.tokens for r in other]
    alone = LLM(folder, dtype="float32", num_blocks=96, block_size=block).generate([prompts[3]], [params[3]], max_tokens=12)
    assert alone[0].tokens == batched[3].tokens
    assert batched[0].tokens == _plain_greedy(cfg, weights, prompts[0], 12)
    reseeded = LLM(folder, dtype="float32", num_blocks=96, block_size=block).generate(
        [prompts[1]], [SamplingParams(temperature=0.8, seed=9)], max_tokens=12)
    assert reseeded[0].tokens != batched[1].tokens


def test_tiny_b_workload_to_two_hundred_positions(tmp_path):
    """The second tiny workload as it is written down: 4 requests with prompts of 1, 40, 97 and
    150 tokens, prompt portions under a 32-token budget mixed with decoding, pages of 16, two
    requests greedy and two at temperature 0.8 with seeds, every request generating until it
    holds 200 positions, in float32.

    Greedy tokens are the plain model's, all of them.  The sampled tokens are judged along the
    engine's own sequence with the plain model's probabilities: each has a probability that is
    not absurdly small, and their log-probabilities add up to what draws from the plain model's
    distributions give (minus the entropy at each place, within five standard deviations of the
    sum): a sampler with another temperature, or one that draws from other logits, fails that."""
    from mini_infer_amd import Request
    from mini_infer_amd.engine.llm import LLM
    from mini_infer_amd.sampling import SamplingParams

    cfg, block, weights, folder = _folder(tmp_path, "B", 52)
    lengths = (1, 40, 97, 150)
    prompts = [tiny.random_tokens(cfg, n, seed=n) for n in lengths]
    params = [SamplingParams(), SamplingParams(temperature=0.8, seed=7), SamplingParams(),
              SamplingParams(temperature=0.8, seed=8)]
    llm = LLM(folder, dtype="float32", num_blocks=4 * 13, block_size=block, max_num_batched_tokens=32, chunk_size=32,
              max_concurrent=4)
    requests = [Request(p, sp, 200 - len(p)) for p, sp in zip(prompts, params)]
    results = llm.scheduler.run_all(requests)
    assert [len(p) + len(r.tokens) for p, r in zip(prompts, results)] == [200] * 4
    assert all(r.finish_reason == "length" for r in results)
    stats = llm.scheduler.stats
    assert stats["tokens_run"] == 4 * 199 and stats["preemptions"] == 0
    assert llm.runner.num_free_blocks() == 4 * 13
    llm.runner.cache.check()
    for prompt, sp, result in zip(prompts, params, results):
        sequence = list(prompt) + result.tokens
        logits = pl.llama_logits(cfg, weights, np.array(sequence))[len(prompt) - 1 : -1]  # one row per generated token
        if sp.temperature == 0:
            assert result.tokens == logits.argmax(axis=-1).tolist()
            continue
        surprise, spread = 0.0, 0.0
        for row, token in zip(logits, result.tokens):
            dist = pl.sampling_distribution(row, sp.temperature)
            assert dist[token] > 1e-7
            logp = np.log(np.maximum(dist, 1e-300))
            entropy = -(dist * logp).sum()
            surprise += -logp[token] - entropy
            spread += (dist * logp**2).sum() - entropy**2
        assert abs(surprise) < 5 * math.sqrt(spread), (surprise, math.sqrt(spread))
        # the yardstick bites: judged at temperature 0.4 or 1.6 the same tokens do not pass
        # (where there are enough of them: the request with the long prompt draws only 50)
        for other in (0.4, 1.6) if len(result.tokens) >= 100 else ():
            off, off_spread = 0.0, 0.0
            for row, token in zip(logits, result.tokens):
                dist = pl.sampling_distribution(row, other)
                logp = np.log(np.maximum(dist, 1e-300))
                entropy = -(dist * logp).sum()
                off += -logp[token] - entropy
                off_spread += (dist * logp**2).sum() - entropy**2
            assert abs(off) > 5 * math.sqrt(off_spread)


@pytest.mark.parametrize("seed", range(6))
def test_random_loads_on_the_real_engine_generate_what_the_plain_model_generates(tmp_path, seed):
    """Random loads (prompt lengths, token counts, pool from tight to roomy, budget, portion
    size, seats) through `LLM` in float32 with the engine's own sampling on the device, ids
    read a step late: every request that ends by itself has the plain model's greedy tokens,
    a cancelled one a prefix of them, and the pool is whole afterwards."""
    from mini_infer_amd.engine.llm import LLM

    cfg, block, weights, folder = _folder(tmp_path, "A", 70 + seed)
    rng = np.random.default_rng(500 + seed)
    num_blocks = int(rng.integers(14, 60))
    llm = LLM(folder, dtype="float32", num_blocks=num_blocks, block_size=block,
              max_num_batched_tokens=int(rng.integers(8, 48)), chunk_size=int(rng.integers(4, 48)),
              max_concurrent=int(rng.integers(1, 6)), decode_headroom_blocks=int(rng.integers(0, 3)))
    prompts = [tiny.random_tokens(cfg, int(rng.integers(1, 40)), seed=seed * 50 + i) for i in range(int(rng.integers(2, 8)))]
    new_tokens = int(rng.integers(1, 12))
    results = llm.generate(prompts, max_tokens=new_tokens)
    for prompt, result in zip(prompts, results):
        expected = _plain_greedy(cfg, weights, prompt, new_tokens)
        if result.finish_reason == "cancelled":
            assert result.tokens == expected[: len(result.tokens)]
        else:
            assert result.tokens == expected and result.finish_reason == "length"
    llm.runner.cache.check()
    assert llm.runner.num_free_blocks() == num_blocks


def test_preemption_on_the_real_engine_keeps_outputs(tmp_path):
    from mini_infer_amd.engine.llm import LLM

    cfg, block, weights, folder = _folder(tmp_path, "A", 53)
    prompts = [tiny.random_tokens(cfg, 12, seed=s) for s in (1, 2, 3)]
    llm = LLM(folder, dtype="float32", num_blocks=14, block_size=block, decode_headroom_blocks=0)
    results = llm.generate(prompts, max_tokens=14)
    assert llm.scheduler.stats["preemptions"] >= 1
    for prompt, result in zip(prompts, results):
        assert result.tokens == _plain_greedy(cfg, weights, prompt, 14)
    assert llm.runner.num_free_blocks() == 14


def test_asynchronous_sampling_gives_the_tokens_of_synchronous_sampling(tmp_path):
    """Ids read one step late: the same tokens and finish reasons as reading them at once, with
    requests that end by end-of-sequence (seen a step late), by length (1 and more tokens),
    sampled and greedy ones, so few pages that requests are preempted, and a cancelled one."""
    from mini_infer_amd import ContinuousScheduler, ModelRunner, Request, SamplingParams

    cfg, block, weights, folder = _folder(tmp_path, "B", 62)
    prompts = [tiny.random_tokens(cfg, n, seed=20 + n) for n in (3, 40, 17, 64, 9, 31)]
    # an end-of-sequence id that greedy decoding of the first prompts runs into after a few tokens
    greedy = _plain_greedy(cfg, weights, prompts[1], 10)
    eos = greedy[4]
    limits = [9, 30, 1, 12, 2, 25]
    params = [SamplingParams(), SamplingParams(), SamplingParams(temperature=0.9, seed=3),
              SamplingParams(temperature=0.7, seed=4, top_k=40), SamplingParams(), SamplingParams(ignore_eos=True)]

    def run(async_sampling, num_blocks):
        runner = ModelRunner.from_pretrained(folder, dtype="float32", num_blocks=num_blocks, block_size=block)
        scheduler = ContinuousScheduler(runner, max_concurrent=4, chunk_size=16, max_num_batched_tokens=24,
                                        decode_headroom_blocks=0, eos_token_id=eos, async_sampling=async_sampling)
        assert scheduler.async_sampling is async_sampling
        results = scheduler.run_all([Request(p, sp, n) for p, sp, n in zip(prompts, params, limits)])
        assert runner.num_free_blocks() == num_blocks and not scheduler.has_work()
        runner.cache.check()
        return [(r.tokens, r.finish_reason) for r in results], scheduler.stats

    for num_blocks in (64, 7):  # plenty of pages; so few that requests are preempted and recomputed
        late, late_stats = run(True, num_blocks)
        at_once, _ = run(False, num_blocks)
        assert late == at_once, f"{num_blocks} pages"
        if num_blocks == 7:
            assert late_stats["preemptions"] >= 1
    assert at_once[1] == (greedy[:4], "stop")  # the end-of-sequence id is not emitted
    assert at_once[2][1] == "length" and len(at_once[2][0]) == 1
    assert len(at_once[5][0]) == 25  # ignore_eos runs to its length
    # streaming and cancelling while ids are in flight
    runner = ModelRunner.from_pretrained(folder, dtype="float32", num_blocks=64, block_size=block)
    scheduler = ContinuousScheduler(runner, async_sampling=True)
    keep = scheduler.submit(Request(prompts[0], SamplingParams(ignore_eos=True), 8))
    drop = scheduler.submit(Request(prompts[2], SamplingParams(ignore_eos=True), 50))
    streamed = []
    for step in keep.stream():
        streamed += list(step.tokens)
        if len(streamed) == 3:
            drop.cancel()
    assert streamed == keep.wait().tokens and len(streamed) == 8
    assert drop.wait().finish_reason == "cancelled" and runner.num_free_blocks() == 64


def test_command_line_generates(tmp_path):
    cfg, block, weights, folder = _folder(tmp_path, "A", 54)
    prompt = tiny.random_tokens(cfg, 6, seed=1)
    done = subprocess.run(
        [sys.executable, "-m", "mini_infer_amd", "generate", "--model", str(folder), "--prompt-ids",
         " ".join(map(str, prompt)), "--max-tokens", "5", "--dtype", "float32", "--block-size", str(block),
         "--num-blocks", "32"],
        cwd=ROOT, capture_output=True, text=True, timeout=110)
    assert done.returncode == 0, done.stderr[-2000:]
    record = json.loads(done.stdout.strip().splitlines()[-1])
    assert record["tokens"] == _plain_greedy(cfg, weights, prompt, 5) and record["finish_reason"] == "length"


# -- the replay program ----------------------------------------------------------------


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_run_program(tmp_path, dtype):
    """bin/trace_run as a user runs it: JSON steps on stdin, <step>.f32 files, `done <step>` lines."""
    cfg, block, weights, folder = _folder(tmp_path, "B", 55)
    requests = {f"r{i}": tiny.random_tokens(cfg, n, seed=i) for i, n in enumerate((40, 70, 33, 64, 50))}
    expected = {rid: ru.oracle(cfg, weights, t) for rid, t in requests.items()}
    schedule = ru.schedule_mixed(requests, seed=5)
    # each request's count rounded up to a multiple of 64
    fed = {rid: 0 for rid in requests}
    live, peak = set(), 0
    lines, wanted = [], []
    for number, step in enumerate(schedule):
        entries = []
        for rid, count in step["feed"].items():
            want = [count - 1] if count > 1 else [0]
            entries.append({"id": rid, "tokens": requests[rid][fed[rid]: fed[rid] + count], "want": want})
            wanted.append((number, rid, fed[rid] + want[0]))
            fed[rid] += count
            live.add(rid)
        peak = max(peak, sum(-(-fed[r] // 64) * 64 for r in live))
        live -= set(step["end"])
        lines.append(json.dumps({"step": number, "entries": entries, "end": step["end"]}))
    out_dir = tmp_path / "out"
    done = subprocess.run(
        [os.path.join(ROOT, "bin", "trace_run"), "--model", str(folder), "--dtype", dtype, "--out", str(out_dir),
         "--max-tokens", str(peak)],
        input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=110)
    assert done.returncode == 0, done.stderr[-2000:]
    assert done.stdout.split("\n")[:-1] == [f"done {n}" for n in range(len(schedule))]
    at = {}
    for number, rid, position in wanted:
        rows = np.fromfile(out_dir / f"{number}.f32", dtype="<f4").reshape(-1, cfg["vocab_size"])
        row = rows[at.get(number, 0)]
        at[number] = at.get(number, 0) + 1
        ru.assert_close(row[None], expected[rid][position][None], dtype, f"step {number} {rid}@{position}")


def test_make_trace_feeds_trace_run_and_a_request_left_live_is_no_error(tmp_path):
    """`python -m mini_infer_amd make-trace` prints what `bin/trace_run` reads; a trace that never
    ends its last request still ends with exit code 0 (the program gives the pages back itself
    and then finds the pool whole)."""
    cfg, block, weights, folder = _folder(tmp_path, "A", 54)
    made = subprocess.run(
        [sys.executable, "-m", "mini_infer_amd", "make-trace", "--family", "mixed", "--lengths", "37,12,20",
         "--vocab-size", str(cfg["vocab_size"]), "--seed", "3", "--tail", "6"],
        capture_output=True, text=True, timeout=60, cwd=ROOT)
    assert made.returncode == 0, made.stderr[-2000:]
    lines = [json.loads(line) for line in made.stdout.splitlines()]
    assert sum(len(e["tokens"]) for line in lines for e in line["entries"]) == 37 + 12 + 20
    lines[-1]["end"] = []  # the last request is never ended
    out_dir = tmp_path / "out"
    done = subprocess.run(
        [os.path.join(ROOT, "bin", "trace_run"), "--model", str(folder), "--dtype", "float32", "--out", str(out_dir),
         "--max-tokens", "192", "--block-size", str(block)],
        input="\n".join(json.dumps(line) for line in lines) + "\n", capture_output=True, text=True, timeout=110)
    assert done.returncode == 0, done.stderr[-2000:]
    assert done.stdout.split("\n")[:-1] == [f"done {n}" for n in range(len(lines))]
    # the logits of the first step's first entry are the plain model's
    first = lines[0]["entries"][0]
    rows = np.fromfile(out_dir / "0.f32", dtype="<f4").reshape(-1, cfg["vocab_size"])
    expected = pl.llama_logits(cfg, weights, np.array(first["tokens"]))
    ru.assert_close(rows[: len(first["tokens"])], expected, "float32", "make-trace step 0")


# -- long decoding, first tokens -----------------------------------------------------------


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(tmp_path, dtype):
    """A short prompt and 380 tokens one by one: far past the rope's original length
    (64 for this configuration), across many pages."""
    from mini_infer_amd.engine import ModelRunner

    cfg, block, weights, folder = _folder(tmp_path, "B", 56)
    requests = {"long": tiny.random_tokens(cfg, 400, seed=9)}
    expected = {"long": ru.oracle(cfg, weights, requests["long"])}
    schedule = ru.schedule_prefill_then_decode(requests, tail=380)
    runner = ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=26, block_size=block)
    got = ru.run_schedule(runner, requests, schedule)
    ru.assert_close(got["long"], expected["long"], dtype, "long decoding")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "C"])
def test_first_tokens_of_a_sequence(tmp_path, name, dtype):
    from mini_infer_amd.engine import ModelRunner

    cfg, block, weights, folder = _folder(tmp_path, name, 57)
    runner = ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=16, block_size=block)
    for length in (1, 2, 3):
        requests = {f"s{length}": tiny.random_tokens(cfg, length, seed=length)}
        expected = ru.oracle(cfg, weights, requests[f"s{length}"])
        token_by_token = [{"feed": {f"s{length}": 1}} for _ in range(length)]
        token_by_token[-1]["end"] = [f"s{length}"]
        got = ru.run_schedule(runner, requests, token_by_token)
        ru.assert_close(got[f"s{length}"], expected, dtype, f"{name} first {length} tokens")


@pytest.mark.parametrize("dtype", DTYPES)
def test_graph_replays_equal_eager_steps_with_eager_work_between(tmp_path, dtype):
    """Decode steps replayed as HIP graphs give the logits of the same steps run eagerly,
    on every replay, with prompt portions (eager work) and synchronizations in between,
    for batches that fill a bucket and batches that are padded."""
    from mini_infer_amd.engine import ModelRunner, StepEntry

    cfg, block, weights, folder = _folder(tmp_path, "B", 59)
    graphed = ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=64, block_size=block, cuda_graph=True)
    eager = ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=64, block_size=block, cuda_graph=False)
    assert graphed.decode_graphs is not None and eager.decode_graphs is None
    rng = np.random.default_rng(0)
    live: list[str] = []
    limit = 2e-5 if dtype == "float32" else 0.05
    for round_ in range(6):
        # eager work: a new request's prompt in two portions, beside nothing else
        rid = f"g{round_}"
        prompt = tiny.random_tokens(cfg, int(rng.integers(20, 60)), seed=round_)
        for runner in (graphed, eager):
            runner.step([StepEntry(rid, prompt[:7], [])])
            runner.step([StepEntry(rid, prompt[7:], [len(prompt) - 8])])
        live.append(rid)
        # several decode steps of all live requests (1, 2, 3, ... rows: padded buckets too)
        for _ in range(5):
            tokens = {r: int(rng.integers(0, cfg["vocab_size"])) for r in live}
            outs = []
            for runner in (graphed, eager):
                logits = runner.step([StepEntry(r, [tokens[r]], [0]) for r in live])
                outs.append(logits.cpu().numpy().copy())
            torch.cuda.synchronize()
            assert np.abs(outs[0] - outs[1]).max() < limit, f"round {round_}"
    assert graphed.decode_graphs.replays == 30 and len(graphed.decode_graphs.graphs) >= 3
    for runner in (graphed, eager):
        for rid in live:
            runner.free_request(rid)
        runner.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["B", "D", "E"])
def test_small_steps_with_portions_are_recorded_by_bucket_and_replayed_with_other_divisions(tmp_path, name, dtype):
    """Steps of a few tokens that are not single tokens only (a prompt's portion beside decoded
    tokens, two short prompts, a portion alone) are recorded once per (tokens, requests) bucket and
    replayed with whatever division of the tokens among the requests the next step has: the
    boundaries live on the device only.  Every wanted row is compared with the plain model; the
    same bucket is replayed with four different divisions, a recorded single-token step and eager
    work of another kind run in between, and a request that ends frees pages that a later
    request's portion then uses."""
    from mini_infer_amd.engine import ModelRunner, StepEntry

    cfg, block, weights, folder = _folder(tmp_path, name, 81)
    lengths = {"a": 40, "b": 23, "c": 31, "d": 12, "e": 50}
    requests = {rid: tiny.random_tokens(cfg, n, seed=30 + n) for rid, n in lengths.items()}
    expected = {rid: ru.oracle(cfg, weights, t) for rid, t in requests.items()}
    runner = ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=-(-100 // block) + 4, block_size=block, max_concurrent=4)
    fed = {rid: 0 for rid in requests}

    def step(*parts):
        """parts: (request, tokens to feed, whether the last of them wants logits)"""
        entries, wanted = [], []
        for rid, count, wants in parts:
            tokens = requests[rid][fed[rid] : fed[rid] + count]
            assert len(tokens) == count
            entries.append(StepEntry(rid, tokens, [count - 1] if wants else []))
            fed[rid] += count
            if wants:
                wanted.append((rid, fed[rid] - 1))
        logits = runner.step(entries).cpu().numpy()
        assert logits.shape[0] == len(wanted)
        for row, (rid, position) in enumerate(wanted):
            ru.assert_close(logits[row : row + 1], expected[rid][position : position + 1], dtype, f"{name} {rid}[{position}]")

    graphs = runner.decode_graphs
    step(("a", 10, False), ("b", 7, True))  # 17 tokens, 2 requests: bucket (32, 4)
    assert list(graphs.graphs) == [(32, 4, 16)] and graphs.mixed_replays == 1
    step(("a", 1, True), ("b", 1, True), ("c", 9, True))  # 11 tokens, 3 requests: bucket (16, 4)
    step(("a", 1, True), ("c", 11, False), ("d", 3, True))  # the same bucket, another division
    step(("a", 1, True), ("b", 1, True), ("c", 1, True), ("d", 1, True))  # single tokens: their own recorded step
    torch.randn(64, 64, device=DEV) @ torch.randn(64, 64, device=DEV)  # eager work of another kind
    step(("b", 1, True), ("c", 5, True), ("d", 1, False))  # (16, 4) again: one request wants nothing
    step(("d", 7, True))  # a portion alone, 7 tokens, 1 request: bucket (16, 2)
    assert fed["d"] == lengths["d"]
    runner.free_request("d")
    step(("e", 16, False), ("a", 1, True))  # 17 tokens: (32, 4) again, the new request on d's pages
    step(("e", 14, True), ("a", 2, True), ("b", 2, True), ("c", 2, True))  # 20 tokens, 4 requests, none to spare: (32, 8)
    step(("e", 16, True))  # exactly the bucket's tokens: (16, 1)
    step(("a", 1, True), ("b", 1, False))  # single tokens, but one of them wants nothing: (16, 4) once more
    assert set(graphs.graphs) == {(32, 4, 16), (16, 4, 16), (4, 16), (16, 2, 16), (32, 8, 16), (16, 1, 16)}
    assert graphs.mixed_replays == 9 and graphs.replays == 1
    # a step of more tokens than the largest bucket, or one that wants two rows of a request, is launched kernel by kernel
    before = graphs.mixed_replays
    runner.step([StepEntry("a", requests["a"][fed["a"] : fed["a"] + 3], [0, 2])])
    assert graphs.mixed_replays == before
    for rid in ("a", "b", "c", "e"):
        runner.free_request(rid)
    runner.cache.check()
    assert runner.num_free_blocks() == runner.num_blocks


@pytest.mark.parametrize("cuda_graph", [True, False])
def test_tokens_left_on_the_device_give_the_steps_of_tokens_from_the_host(tmp_path, cuda_graph):
    """A decode step whose tokens are still on the device (`device_row`) equals the step fed
    from the host; in changing row order, with rows left out, beside a prompt portion."""
    from mini_infer_amd.engine import ModelRunner, StepEntry
    from mini_infer_amd.sampling import SamplingParams, sample_tokens

    cfg, block, weights, folder = _folder(tmp_path, "B", 61)
    runners = [ModelRunner.from_pretrained(folder, dtype="float32", num_blocks=64, block_size=block, cuda_graph=cuda_graph)
               for _ in range(2)]
    by_device, by_host = runners
    ids = ["p", "q", "r"]
    greedy = [SamplingParams()] * 3
    for n, rid in enumerate(ids):
        prompt = tiny.random_tokens(cfg, 9 + 5 * n, seed=n)
        for runner in runners:
            runner.step([StepEntry(rid, prompt, [])])
    first = [3, 5, 7]
    device_logits = by_device.step([StepEntry(r, [t], [0]) for r, t in zip(ids, first)])
    host_logits = by_host.step([StepEntry(r, [t], [0]) for r, t in zip(ids, first)])
    for step in range(6):
        sampled = sample_tokens(device_logits, greedy, [0] * 3, [step] * 3)  # stays on the device
        on_host = sample_tokens(host_logits, greedy, [0] * 3, [step] * 3).tolist()
        order = [(step + i) % 3 for i in range(3)]  # the rows change places from step to step
        entries_d = [StepEntry(ids[j], [0], [0], device_row=j) for j in order]
        entries_h = [StepEntry(ids[j], [on_host[j]], [0]) for j in order]
        if step == 3:  # a new request's prompt beside the decode tokens: not a pure decode step
            extra = StepEntry("new", tiny.random_tokens(cfg, 6, seed=9), [5])
            entries_d.append(extra), entries_h.append(extra)
        device_logits = by_device.step(entries_d, device_tokens=sampled)
        host_logits = by_host.step(entries_h)
        assert torch.equal(device_logits, host_logits), f"step {step}"
        inverse = [order.index(j) for j in range(3)]  # back to the order of `ids` for the next sample
        device_logits, host_logits = device_logits[inverse], host_logits[inverse]
    with pytest.raises(ValueError, match="device_row"):
        by_device.step([StepEntry("p", [0], [0], device_row=0)])
    with pytest.raises(ValueError, match="device_row"):
        by_device.step([StepEntry("p", [0, 1], [0], device_row=0)], device_tokens=sampled)


@pytest.mark.parametrize("name", ["A", "C", "D", "E"])
def test_no_step_falls_back_to_torch_operations(tmp_path, monkeypatch, name):
    """What flows between parts in place of a tensor (`PartialSums`, `AttentionPieces`,
    `ScaledRows`) can always be turned into one by `finish()`, a chain of torch operations meant
    for parts that know none of them.  The built-in parts never need it: a norm asks the part
    that follows before it leaves the rows' factors to it.  Portions, single tokens alone and
    eight at once (launched kernel by kernel, so that every call is seen), head sizes the
    folded kernels take (D) and do not take (A, C, E)."""
    from mini_infer_amd import ops
    from mini_infer_amd.engine import ModelRunner, StepEntry

    calls = []
    for kind in (ops.PartialSums, ops.AttentionPieces, ops.ScaledRows):
        monkeypatch.setattr(kind, "finish", lambda self, kind=kind: calls.append(kind.__name__) or pytest.fail(f"{kind.__name__}.finish() ran"))
    cfg, block, weights, folder = _folder(tmp_path, name, 77)
    runner = ModelRunner.from_pretrained(folder, dtype="bfloat16", num_blocks=64, block_size=block, max_concurrent=8, cuda_graph=False)
    prompts = {f"n{i}": tiny.random_tokens(cfg, 9 + 5 * i, seed=i) for i in range(8)}
    runner.step([StepEntry(rid, t[:-3], []) for rid, t in prompts.items()])
    for k in (3, 2):
        runner.step([StepEntry("n0", prompts["n0"][-k : len(prompts["n0"]) - k + 1], [0])])
    runner.step([StepEntry(rid, t[-3:-2], [0]) for rid, t in list(prompts.items())[1:]])
    runner.step([StepEntry(rid, t[-1:] if rid == "n0" else t[-2:-1], [0]) for rid, t in prompts.items()])
    assert calls == []


def test_model_with_a_host_looping_part_is_not_graphed(tmp_path):
    """A model holding a part that does not declare itself `graph_safe` (here a pass-through
    feed-forward defined in the test) gets no decode graphs: its single-token steps run eagerly."""
    import copy
    import dataclasses

    from mini_infer_amd.engine import ModelRunner, StepEntry
    from mini_infer_amd.models.spec import LayerSpec
    from mini_infer_amd.parts import FeedForward
    from mini_infer_amd.registry import ARCHITECTURES, FEED_FORWARDS

    class Nothing(FeedForward):
        def forward(self, x, ctx):
            assert len(ctx.host_seq_lens) == ctx.num_requests  # the host lists a looping part would read
            return torch.zeros_like(x)

    FEED_FORWARDS.register("nothing", lambda desc, dtype_, device, shared=None: Nothing(dtype_, device))

    def with_toy(spec):
        layers = list(spec.layers)
        block = copy.deepcopy(layers[1].block)
        block["feed_forward"] = {"kind": "nothing"}
        layers[1] = LayerSpec(layers[1].prefix, block)
        return dataclasses.replace(spec, layers=layers)

    _register_variant("NotGraphedTestLM", with_toy)
    try:
        cfg = dict(tiny.TINY_A, architectures=["NotGraphedTestLM"])
        weights = tiny.make_weights(cfg, 59)
        for n in ("gate", "up", "down"):
            del weights[f"model.layers.1.mlp.{n}_proj.weight"]
        folder = tiny.write_model_dir(tmp_path / "notgraphed", cfg, weights)
        runner = ModelRunner.from_pretrained(folder, dtype="bfloat16", num_blocks=8, block_size=4)
        assert not runner.model.graph_safe and runner.decode_graphs is None
        runner.step([StepEntry("a", [1, 2, 3], [2])])
        for token in (4, 5, 6):
            assert runner.step([StepEntry("a", [token], [0])]).shape == (1, cfg["vocab_size"])
        # the same folder's plain Llama sibling does record its decode steps
        plain_cfg, _, _, plain_folder = _folder(tmp_path, "A", 59)
        graphed = ModelRunner.from_pretrained(plain_folder, dtype="bfloat16", num_blocks=8, block_size=4)
        graphed.step([StepEntry("a", [1, 2, 3], [2])])
        graphed.step([StepEntry("a", [4], [0])])
        assert graphed.decode_graphs is not None and graphed.decode_graphs.replays == 1
    finally:
        ARCHITECTURES.unregister("NotGraphedTestLM")
        FEED_FORWARDS.unregister("nothing")


def test_step_refuses_bad_batches(tmp_path):
    from mini_infer_amd.engine import ModelRunner, StepEntry
    from mini_infer_amd.exceptions import OutOfMemoryError

    cfg, block, weights, folder = _folder(tmp_path, "A", 58)
    runner = ModelRunner.from_pretrained(folder, dtype="float32", num_blocks=4, block_size=block)
    with pytest.raises(ValueError, match="token ids"):
        runner.step([StepEntry("a", [cfg["vocab_size"]], [0])])
    with pytest.raises(ValueError, match="twice"):
        runner.step([StepEntry("a", [1], [0]), StepEntry("a", [2], [0])])
    with pytest.raises(ValueError, match="outside"):
        runner.step([StepEntry("a", [1, 2], [2])])
    with pytest.raises(OutOfMemoryError):
        runner.step([StepEntry("a", [1] * 17, [])])
    assert not runner.has_request("a") and runner.num_free_blocks() == 4  # nothing changed
    assert runner.step([StepEntry("a", [1, 2, 3], [])]).shape == (0, cfg["vocab_size"])
    assert runner.cache.length("a") == 3


# -- the model as data: order lists, windows, a toy mixer from outside -----------------------


def _register_variant(name, transform):
    """An architecture defined here: Llama's spec with `transform` applied to it."""
    from mini_infer_amd.config import ModelConfig
    from mini_infer_amd.models.llama import llama_spec
    from mini_infer_amd.models.spec import Architecture
    from mini_infer_amd.registry import ARCHITECTURES

    ARCHITECTURES.register(name, Architecture(name, ModelConfig.from_dict, lambda cfg: transform(llama_spec(cfg))))


@pytest.mark.parametrize("dtype", DTYPES)
def test_order_list_names_a_layer_twice_and_reads_another_cache(tmp_path, dtype):
    import dataclasses

    from mini_infer_amd.engine import ModelRunner
    from mini_infer_amd.models.spec import LayerCall
    from mini_infer_amd.registry import ARCHITECTURES

    order = [LayerCall(0), LayerCall(1), LayerCall(0), LayerCall(1, reads_cache_of=1)]
    _register_variant("LoopedTestLM", lambda spec: dataclasses.replace(spec, order=order))
    try:
        cfg = dict(tiny.TINY_A, architectures=["LoopedTestLM"])
        weights = tiny.make_weights(cfg, 60)
        folder = tiny.write_model_dir(tmp_path / "looped", cfg, weights)
        requests = {"x": tiny.random_tokens(cfg, 45, 1), "y": tiny.random_tokens(cfg, 30, 2)}
        plain_order = [(0, None), (1, None), (0, None), (1, 1)]
        expected = {r: ru.oracle(cfg, weights, t, order=plain_order) for r, t in requests.items()}
        runner = ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=24, block_size=4)
        assert len(runner.cache.groups) == 1 and runner.cache.groups[0].calls == [0, 1, 2]
        got = ru.run_schedule(runner, requests, ru.schedule_mixed(requests, seed=2, tail=8))
        for rid in requests:
            ru.assert_close(got[rid], expected[rid], dtype, f"looped {rid}")
    finally:
        ARCHITECTURES.unregister("LoopedTestLM")


@pytest.mark.parametrize("dtype", DTYPES)
def test_layers_with_and_without_a_window_have_page_groups_of_their_own(tmp_path, dtype):
    import copy
    import dataclasses

    from mini_infer_amd.cache import RELEASED
    from mini_infer_amd.engine import ModelRunner
    from mini_infer_amd.models.spec import LayerSpec
    from mini_infer_amd.registry import ARCHITECTURES

    def windowed(spec):
        layers = []
        for i, layer in enumerate(spec.layers):
            block = copy.deepcopy(layer.block)
            block["mixer"]["window"] = 6 if i % 2 == 0 else None
            layers.append(LayerSpec(layer.prefix, block))
        return dataclasses.replace(spec, layers=layers)

    _register_variant("WindowedTestLM", windowed)
    try:
        cfg = dict(tiny.TINY_B, architectures=["WindowedTestLM"])
        weights = tiny.make_weights(cfg, 61)
        folder = tiny.write_model_dir(tmp_path / "windowed", cfg, weights)
        requests = {"x": tiny.random_tokens(cfg, 61, 1), "y": tiny.random_tokens(cfg, 38, 2)}
        expected = {r: ru.oracle(cfg, weights, t, window=[6, None, 6]) for r, t in requests.items()}
        runner = ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=10, block_size=4)
        groups = {g.window: g for g in runner.cache.groups}
        assert sorted(groups, key=str) == [6, None] and groups[6].calls == [0, 2] and groups[None].calls == [1]
        from mini_infer_amd.engine import StepEntry

        # x alone first: after 30 tokens the windowed group has given back all but two or three pages
        logits = runner.step([StepEntry("x", requests["x"][:30], list(range(30)))]).cpu().numpy()
        ru.assert_close(logits, expected["x"][:30], dtype, "windowed x[:30]")
        assert groups[6].tables["x"][:6] == [RELEASED] * 6
        assert groups[6].pool.num_free == 10 - 2 and groups[None].pool.num_free == 10 - 8
        rest = {"x": requests["x"][30:], "y": requests["y"]}
        # the full group has 2 pages left: y must wait there, so feed y in the windowed order only after x ends
        got_x = runner.step([StepEntry("x", rest["x"][:8], list(range(8)))]).cpu().numpy()
        ru.assert_close(got_x, expected["x"][30:38], dtype, "windowed x[30:38]")
        runner.free_request("x")
        got = ru.run_schedule(runner, {"y": requests["y"]}, ru.schedule_portions({"y": requests["y"]}, seed=1))
        ru.assert_close(got["y"], expected["y"], dtype, "windowed y")
        runner.cache.check()
        assert all(g.pool.num_free == 10 for g in runner.cache.groups)
        if dtype == "float32":
            # through the scheduler: portions under a small budget beside single tokens (recorded
            # steps with portions in them), pages the window has passed given back on the way
            from mini_infer_amd.engine.llm import LLM

            llm = LLM(folder, dtype=dtype, num_blocks=24, block_size=4, max_num_batched_tokens=24, chunk_size=16, max_concurrent=3)
            prompts = [tiny.random_tokens(cfg, n, seed=90 + n) for n in (21, 5, 34, 12)]
            for prompt, result in zip(prompts, llm.generate(prompts, max_tokens=7)):
                sequence = list(prompt)
                for _ in range(7):
                    sequence.append(pl.greedy(pl.llama_logits(cfg, weights, np.array(sequence), window=[6, None, 6])[-1]))
                assert result.tokens == sequence[len(prompt):] and result.finish_reason == "length"
            assert llm.runner.decode_graphs.mixed_replays > 0 and llm.runner.decode_graphs.replays > 0
            llm.runner.cache.check()
            assert all(g.pool.num_free == 24 for g in llm.runner.cache.groups)
    finally:
        ARCHITECTURES.unregister("WindowedTestLM")


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_mixer_with_state_registers_builds_and_steps(tmp_path, dtype):
    """A mixer defined here, with state of fixed size per request (a decaying sum of its
    inputs) and no pages, is registered, built from a layer description, loaded from a
    checkpoint by name, and stepped in portions and mixed batches: no framework file changes."""
    import copy
    import dataclasses

    from mini_infer_amd.engine import ModelRunner
    from mini_infer_amd.models.spec import LayerSpec
    from mini_infer_amd.parts import CacheNeeds, Mixer, ParamSpec, StateNeeds
    from mini_infer_amd.registry import ARCHITECTURES, MIXERS

    hidden = tiny.TINY_A["hidden_size"]
    decay = 0.75

    class DecayingSum(Mixer):
        def param_specs(self, prefix):
            return {prefix + "mix.weight": ParamSpec((hidden, hidden))}

        def load_params(self, prefix, get):
            self.weight = get(prefix + "mix.weight")

        def cache_needs(self, page_size):
            return CacheNeeds(state=StateNeeds((hidden,), torch.float32))

        def forward(self, x, ctx, cache, writes_cache=True):
            out = torch.empty_like(x)
            for b, slot in enumerate(ctx.host_state_slots):
                state = cache.state[slot]
                for t in range(ctx.host_cu_seqlens_q[b], ctx.host_cu_seqlens_q[b + 1]):
                    state = decay * state + x[t].float()
                    out[t] = (self.weight.float() @ state).to(x.dtype)
                cache.state[slot] = state
            return out

    MIXERS.register("decaying_sum", lambda desc, dtype_, device, shared=None: DecayingSum(dtype_, device))

    def with_toy(spec):
        layers = list(spec.layers)
        block = copy.deepcopy(layers[1].block)
        block["mixer"] = {"kind": "decaying_sum"}
        layers[1] = LayerSpec(layers[1].prefix, block)
        return dataclasses.replace(spec, layers=layers)

    _register_variant("ToyStateTestLM", with_toy)
    try:
        cfg = dict(tiny.TINY_A, architectures=["ToyStateTestLM"])
        weights = tiny.make_weights(cfg, 62)
        for n in "qkvo":
            del weights[f"model.layers.1.self_attn.{n}_proj.weight"]
        rng = np.random.default_rng(3)
        weights["model.layers.1.self_attn.mix.weight"] = tiny.bf16_round(rng.standard_normal((hidden, hidden)) / 16)
        folder = tiny.write_model_dir(tmp_path / "toy", cfg, weights)

        def plain(tokens):
            """Layer 0 as Llama's, layer 1 with the decaying sum in place of attention."""
            eps = cfg["rms_norm_eps"]
            r = pl.embedding(weights["model.embed_tokens.weight"], np.array(tokens))
            cos, sin = pl.rope_tables(np.arange(len(tokens)), pl.config_inv_freq(cfg))
            p = "model.layers.0."
            a, _ = pl.attention_layer(
                pl.rms_norm(r, weights[p + "input_layernorm.weight"], eps),
                *(weights[p + f"self_attn.{n}_proj.weight"] for n in "qkvo"), cos, sin, 4, 2, 16)
            r = r + a
            r = r + pl.swiglu(pl.rms_norm(r, weights[p + "post_attention_layernorm.weight"], eps),
                              *(weights[p + f"mlp.{n}_proj.weight"] for n in ("gate", "up", "down")))
            p = "model.layers.1."
            h = pl.rms_norm(r, weights[p + "input_layernorm.weight"], eps)
            if dtype == "bfloat16":
                h = tiny.bf16_round(h).astype(np.float64)
            state, mixed = np.zeros(hidden), []
            for row in h:
                state = decay * state + row
                mixed.append(weights[p + "self_attn.mix.weight"].astype(np.float64) @ state)
            r = r + np.array(mixed)
            r = r + pl.swiglu(pl.rms_norm(r, weights[p + "post_attention_layernorm.weight"], eps),
                              *(weights[p + f"mlp.{n}_proj.weight"] for n in ("gate", "up", "down")))
            return pl.rms_norm(r, weights["model.norm.weight"], eps) @ weights["model.embed_tokens.weight"].astype(np.float64).T

        requests = {f"t{i}": tiny.random_tokens(cfg, n, seed=i) for i, n in enumerate((20, 9, 14, 11, 17))}
        expected = {rid: plain(t) for rid, t in requests.items()}
        runner = ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=24, block_size=4, max_concurrent=4)
        caches = runner.cache.layer_caches()
        assert caches[1].state.shape == (4 + 1, hidden) and caches[1].k_pages is None and caches[0].state is None
        got = ru.run_schedule(runner, requests, ru.schedule_mixed(requests, seed=4, tail=5))
        for rid in requests:
            ru.assert_close(got[rid], expected[rid], dtype, f"toy {rid}")
        runner.cache.check()
        assert runner.cache.states.num_free == 4
    finally:
        ARCHITECTURES.unregister("ToyStateTestLM")
        MIXERS.unregister("decaying_sum")


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_state_mixer_on_device_tensors_alone_is_recorded_and_replayed(tmp_path, dtype):
    """The decaying sum once more, written with device tensors alone (no loop over the step's
    requests on the host) and declared `graph_safe`: its single-token steps are recorded and
    replayed like Llama's.  Three requests decode together in the bucket of four, so one row of
    every replay is padding with slot -1 and must touch no request's state; the run that
    precedes a recording must not advance the state either."""
    import copy
    import dataclasses

    from mini_infer_amd.engine import ModelRunner, StepEntry
    from mini_infer_amd.models.spec import LayerSpec
    from mini_infer_amd.parts import CacheNeeds, Mixer, ParamSpec, StateNeeds
    from mini_infer_amd.registry import ARCHITECTURES, MIXERS

    hidden = tiny.TINY_A["hidden_size"]
    decay = 0.75

    class DecayingSumOnDevice(Mixer):
        graph_safe = True

        def param_specs(self, prefix):
            return {prefix + "mix.weight": ParamSpec((hidden, hidden))}

        def load_params(self, prefix, get):
            self.weight = get(prefix + "mix.weight")

        def cache_needs(self, page_size):
            return CacheNeeds(state=StateNeeds((hidden,), torch.float32))

        def forward(self, x, ctx, cache, writes_cache=True):
            request = ctx.token_request.long()  # [T]
            slots = ctx.state_slots.long()  # [B]; -1 (the spare row) for padding rows
            at = torch.arange(x.shape[0], device=x.device)
            starts = ctx.cu_seqlens_q.long()
            distance = at[:, None] - at[None, :]
            earlier_of_same_request = (request[:, None] == request[None, :]) & (distance >= 0)
            weights = torch.where(earlier_of_same_request, decay ** distance.clamp(min=0).float(), 0.0)
            carried = (decay ** (at - starts[request] + 1).float())[:, None] * cache.state[slots[request]]
            states = weights @ x.float() + carried  # the state after each token
            cache.state[slots] = states[starts[1:] - 1]
            return (states @ self.weight.float().T).to(x.dtype)

    MIXERS.register("decaying_sum_on_device", lambda desc, dtype_, device, shared=None: DecayingSumOnDevice(dtype_, device))

    def with_toy(spec):
        layers = list(spec.layers)
        block = copy.deepcopy(layers[1].block)
        block["mixer"] = {"kind": "decaying_sum_on_device"}
        layers[1] = LayerSpec(layers[1].prefix, block)
        return dataclasses.replace(spec, layers=layers)

    _register_variant("ToyDeviceStateTestLM", with_toy)
    try:
        cfg = dict(tiny.TINY_A, architectures=["ToyDeviceStateTestLM"])
        weights = tiny.make_weights(cfg, 63)
        for n in "qkvo":
            del weights[f"model.layers.1.self_attn.{n}_proj.weight"]
        rng = np.random.default_rng(5)
        weights["model.layers.1.self_attn.mix.weight"] = tiny.bf16_round(rng.standard_normal((hidden, hidden)) / 16)
        folder = tiny.write_model_dir(tmp_path / "toy", cfg, weights)

        def plain(tokens):
            """Layer 0 as Llama's, layer 1 with the decaying sum (a loop over the tokens) in place of attention."""
            eps = cfg["rms_norm_eps"]
            r = pl.embedding(weights["model.embed_tokens.weight"], np.array(tokens))
            cos, sin = pl.rope_tables(np.arange(len(tokens)), pl.config_inv_freq(cfg))
            p = "model.layers.0."
            a, _ = pl.attention_layer(
                pl.rms_norm(r, weights[p + "input_layernorm.weight"], eps),
                *(weights[p + f"self_attn.{n}_proj.weight"] for n in "qkvo"), cos, sin, 4, 2, 16)
            r = r + a
            r = r + pl.swiglu(pl.rms_norm(r, weights[p + "post_attention_layernorm.weight"], eps),
                              *(weights[p + f"mlp.{n}_proj.weight"] for n in ("gate", "up", "down")))
            p = "model.layers.1."
            h = pl.rms_norm(r, weights[p + "input_layernorm.weight"], eps)
            if dtype == "bfloat16":
                h = tiny.bf16_round(h).astype(np.float64)
            state, mixed = np.zeros(hidden), []
            for row in h:
                state = decay * state + row
                mixed.append(weights[p + "self_attn.mix.weight"].astype(np.float64) @ state)
            r = r + np.array(mixed)
            r = r + pl.swiglu(pl.rms_norm(r, weights[p + "post_attention_layernorm.weight"], eps),
                              *(weights[p + f"mlp.{n}_proj.weight"] for n in ("gate", "up", "down")))
            return pl.rms_norm(r, weights["model.norm.weight"], eps) @ weights["model.embed_tokens.weight"].astype(np.float64).T

        prompts, decoded = (13, 6, 9), 7
        requests = {f"d{i}": tiny.random_tokens(cfg, n + decoded, seed=20 + i) for i, n in enumerate(prompts)}
        expected = {rid: plain(t) for rid, t in requests.items()}
        runner = ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=24, block_size=4, max_concurrent=4)
        assert runner.model.graph_safe and runner.decode_graphs is not None
        got = {rid: [] for rid in requests}
        # prompts: the first alone and in two portions, the other two together
        runner.step([StepEntry("d0", requests["d0"][:5], [])])
        got["d0"].append(runner.step([StepEntry("d0", requests["d0"][5:13], list(range(8)))]).cpu().numpy())
        both = runner.step([StepEntry("d1", requests["d1"][:6], [5]), StepEntry("d2", requests["d2"][:9], [8])]).cpu().numpy()
        got["d1"].append(both[:1])
        got["d2"].append(both[1:])
        for k in range(decoded):
            entries = [StepEntry(rid, [requests[rid][n + k]], [0]) for rid, n in zip(requests, prompts)]
            logits = runner.step(entries).cpu().numpy()
            for row, rid in enumerate(requests):
                got[rid].append(logits[row : row + 1])
        assert runner.decode_graphs.replays == decoded and [key for key in runner.decode_graphs.graphs if len(key) == 2] == [(4, 16)]
        ru.assert_close(np.concatenate(got["d0"]), expected["d0"][5:], dtype, "toy on device d0")
        ru.assert_close(np.concatenate(got["d1"]), expected["d1"][5:], dtype, "toy on device d1")
        ru.assert_close(np.concatenate(got["d2"]), expected["d2"][8:], dtype, "toy on device d2")
        for rid in requests:
            runner.free_request(rid)
        runner.cache.check()
        assert runner.cache.states.num_free == 4
    finally:
        ARCHITECTURES.unregister("ToyDeviceStateTestLM")
        MIXERS.unregister("decaying_sum_on_device")


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_routed_feed_forward_registers_builds_and_steps(tmp_path, dtype):
    """A feed-forward defined here that routes each token to one of two small experts (router
    logits and their softmax in float32) takes the place of layer 0's SwiGLU: registered,
    built from a layer description, loaded by name, stepped in mixed batches.  The layer
    beside it keeps its dense feed-forward: one model, two kinds."""
    import copy
    import dataclasses

    from mini_infer_amd.engine import ModelRunner
    from mini_infer_amd.models.spec import LayerSpec
    from mini_infer_amd.parts import FeedForward, ParamSpec
    from mini_infer_amd.registry import ARCHITECTURES, FEED_FORWARDS

    hidden, inner = tiny.TINY_A["hidden_size"], 24

    class OneOfTwo(FeedForward):
        def param_specs(self, prefix):
            specs = {prefix + "router.weight": ParamSpec((2, hidden))}
            for e in range(2):
                specs[prefix + f"experts.{e}.up.weight"] = ParamSpec((inner, hidden))
                specs[prefix + f"experts.{e}.down.weight"] = ParamSpec((hidden, inner))
            return specs

        def load_params(self, prefix, get):
            self.router = get(prefix + "router.weight").float()
            self.up = [get(prefix + f"experts.{e}.up.weight") for e in range(2)]
            self.down = [get(prefix + f"experts.{e}.down.weight") for e in range(2)]

        def forward(self, x, ctx):
            share = torch.softmax(x.float() @ self.router.T, dim=-1)
            choice = share.argmax(dim=-1)
            out = torch.zeros_like(x)
            for e in range(2):
                rows = (choice == e).nonzero().flatten()
                if rows.numel():
                    inside = torch.nn.functional.silu((x[rows].float() @ self.up[e].float().T)).to(x.dtype)
                    result = (inside.float() @ self.down[e].float().T) * share[rows, e : e + 1]
                    out[rows] = result.to(x.dtype)
            return out

    FEED_FORWARDS.register("one_of_two", lambda desc, dtype_, device, shared=None: OneOfTwo(dtype_, device))

    def with_toy(spec):
        layers = list(spec.layers)
        block = copy.deepcopy(layers[0].block)
        block["feed_forward"] = {"kind": "one_of_two"}
        layers[0] = LayerSpec(layers[0].prefix, block)
        return dataclasses.replace(spec, layers=layers)

    _register_variant("ToyRoutedTestLM", with_toy)
    try:
        cfg = dict(tiny.TINY_A, architectures=["ToyRoutedTestLM"])
        weights = tiny.make_weights(cfg, 63)
        for n in ("gate", "up", "down"):
            del weights[f"model.layers.0.mlp.{n}_proj.weight"]
        rng = np.random.default_rng(6)
        p = "model.layers.0.mlp."
        weights[p + "router.weight"] = tiny.bf16_round(rng.standard_normal((2, hidden)) * 2)  # clear choices
        for e in range(2):
            weights[p + f"experts.{e}.up.weight"] = tiny.bf16_round(rng.standard_normal((inner, hidden)) / 6)
            weights[p + f"experts.{e}.down.weight"] = tiny.bf16_round(rng.standard_normal((hidden, inner)) / 6)
        folder = tiny.write_model_dir(tmp_path / "routed", cfg, weights)
        experts_used = set()

        def plain(tokens):
            eps = cfg["rms_norm_eps"]
            r = pl.embedding(weights["model.embed_tokens.weight"], np.array(tokens))
            cos, sin = pl.rope_tables(np.arange(len(tokens)), pl.config_inv_freq(cfg))
            for layer in range(2):
                q = f"model.layers.{layer}."
                a, _ = pl.attention_layer(
                    pl.rms_norm(r, weights[q + "input_layernorm.weight"], eps),
                    *(weights[q + f"self_attn.{n}_proj.weight"] for n in "qkvo"), cos, sin, 4, 2, 16)
                r = r + a
                h = pl.rms_norm(r, weights[q + "post_attention_layernorm.weight"], eps)
                if layer == 1:
                    r = r + pl.swiglu(h, *(weights[q + f"mlp.{n}_proj.weight"] for n in ("gate", "up", "down")))
                    continue
                share = [pl.softmax(row) for row in h @ weights[p + "router.weight"].astype(np.float64).T]
                rows = []
                for row, s in zip(h, share):
                    e = int(np.argmax(s))
                    experts_used.add(e)
                    inside = pl.silu(weights[p + f"experts.{e}.up.weight"].astype(np.float64) @ row)
                    rows.append(weights[p + f"experts.{e}.down.weight"].astype(np.float64) @ inside * s[e])
                r = r + np.array(rows)
            return pl.rms_norm(r, weights["model.norm.weight"], eps) @ weights["model.embed_tokens.weight"].astype(np.float64).T

        requests = {f"r{i}": tiny.random_tokens(cfg, n, seed=10 + i) for i, n in enumerate((18, 7, 13, 22))}
        expected = {rid: plain(t) for rid, t in requests.items()}
        assert experts_used == {0, 1}
        runner = ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=24, block_size=4, max_concurrent=4)
        assert not runner.model.graph_safe  # the toy part does not say it is: its steps are not recorded
        got = ru.run_schedule(runner, requests, ru.schedule_mixed(requests, seed=5, tail=4))
        for rid in requests:
            ru.assert_close(got[rid], expected[rid], dtype, f"routed {rid}")
        runner.cache.check()
    finally:
        ARCHITECTURES.unregister("ToyRoutedTestLM")
        FEED_FORWARDS.unregister("one_of_two")


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_position_encoding_registers_builds_and_steps(tmp_path, dtype):
    """Another position encoding defined here (rotation angles of positions squeezed by a
    factor, with tables it makes itself in torch) is named in the mixer's description of
    layer 1 and used by the framework's attention part as it is."""
    import copy
    import dataclasses

    from mini_infer_amd.engine import ModelRunner
    from mini_infer_amd.models.spec import LayerSpec
    from mini_infer_amd.parts import PositionEncoding, RotaryTables
    from mini_infer_amd.registry import ARCHITECTURES, POSITION_ENCODINGS

    squeeze = 4.0

    class SqueezedRotary(PositionEncoding):
        def __init__(self, desc, dtype_, device):
            super().__init__(dtype_, device)
            self.rotary_dim = int(desc["head_dim"])
            table = pl.inv_freq_default(self.rotary_dim, float(desc["theta"]))
            self.inv_freq = torch.from_numpy(table).to(device)

        def rotary(self, ctx):
            angle = (ctx.positions.float() / squeeze)[:, None] * self.inv_freq[None, :]
            return RotaryTables(torch.cos(angle).contiguous(), torch.sin(angle).contiguous(), self.rotary_dim, False)

    POSITION_ENCODINGS.register("squeezed_rotary", lambda desc, dtype_, device, shared=None: SqueezedRotary(desc, dtype_, device))

    def with_toy(spec):
        layers = list(spec.layers)
        block = copy.deepcopy(layers[1].block)
        block["mixer"]["position"] = dict(block["mixer"]["position"], kind="squeezed_rotary")
        layers[1] = LayerSpec(layers[1].prefix, block)
        return dataclasses.replace(spec, layers=layers)

    _register_variant("ToyPositionTestLM", with_toy)
    try:
        cfg = dict(tiny.TINY_A, architectures=["ToyPositionTestLM"])
        weights = tiny.make_weights(cfg, 64)
        folder = tiny.write_model_dir(tmp_path / "squeezed", cfg, weights)

        def plain(tokens):
            eps = cfg["rms_norm_eps"]
            r = pl.embedding(weights["model.embed_tokens.weight"], np.array(tokens))
            for layer in range(2):
                positions = np.arange(len(tokens)) / (squeeze if layer == 1 else 1.0)
                cos, sin = pl.rope_tables(positions, pl.config_inv_freq(cfg))
                q = f"model.layers.{layer}."
                a, _ = pl.attention_layer(
                    pl.rms_norm(r, weights[q + "input_layernorm.weight"], eps),
                    *(weights[q + f"self_attn.{n}_proj.weight"] for n in "qkvo"), cos, sin, 4, 2, 16)
                r = r + a
                r = r + pl.swiglu(pl.rms_norm(r, weights[q + "post_attention_layernorm.weight"], eps),
                                  *(weights[q + f"mlp.{n}_proj.weight"] for n in ("gate", "up", "down")))
            return pl.rms_norm(r, weights["model.norm.weight"], eps) @ weights["model.embed_tokens.weight"].astype(np.float64).T

        requests = {f"s{i}": tiny.random_tokens(cfg, n, seed=20 + i) for i, n in enumerate((25, 6, 15))}
        expected = {rid: plain(t) for rid, t in requests.items()}
        # the squeeze matters: with plain positions in layer 1 the logits are others
        assert np.abs(expected["s0"] - pl.llama_logits(cfg, weights, np.array(requests["s0"]))).max() > 1e-2
        runner = ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=24, block_size=4, max_concurrent=3)
        got = ru.run_schedule(runner, requests, ru.schedule_mixed(requests, seed=6, tail=5))
        for rid in requests:
            ru.assert_close(got[rid], expected[rid], dtype, f"squeezed {rid}")
        runner.cache.check()
    finally:
        ARCHITECTURES.unregister("ToyPositionTestLM")
        POSITION_ENCODINGS.unregister("squeezed_rotary")


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_distance_penalty_in_place_of_rotation_registers_builds_and_steps(tmp_path, dtype):
    """A position encoding defined here that rotates nothing: it answers the attention part's
    other question, with per-head slopes of a score penalty linear in the distance.  Layer 1
    uses it (its values stay untransposed and the plain kernel runs, in bfloat16 too); layer 0
    keeps its rotation, so the two layers live in page groups of their own."""
    import copy
    import dataclasses

    from mini_infer_amd.engine import ModelRunner
    from mini_infer_amd.models.spec import LayerSpec
    from mini_infer_amd.parts import PositionEncoding
    from mini_infer_amd.registry import ARCHITECTURES, POSITION_ENCODINGS

    class DistancePenalty(PositionEncoding):
        def score_slopes(self, num_heads):
            return torch.tensor([0.5 ** (h + 1) for h in range(num_heads)], dtype=torch.float32, device=self.device)

    POSITION_ENCODINGS.register("distance_penalty", lambda desc, dtype_, device, shared=None: DistancePenalty(dtype_, device))

    def with_toy(spec):
        layers = list(spec.layers)
        block = copy.deepcopy(layers[1].block)
        block["mixer"]["position"] = {"kind": "distance_penalty"}
        layers[1] = LayerSpec(layers[1].prefix, block)
        return dataclasses.replace(spec, layers=layers)

    _register_variant("ToyPenaltyTestLM", with_toy)
    try:
        cfg = dict(tiny.TINY_B, architectures=["ToyPenaltyTestLM"], num_hidden_layers=2)
        weights = tiny.make_weights(cfg, 65)
        folder = tiny.write_model_dir(tmp_path / "penalty", cfg, weights)
        heads, kv_heads, head_dim = 3, 1, 32

        def penalized_attention(h, q_layer):
            t = h.shape[0]
            w = {n: weights[q_layer + f"self_attn.{n}_proj.weight"].astype(np.float64) for n in "qkvo"}
            q = (h @ w["q"].T).reshape(t, heads, head_dim)
            k = (h @ w["k"].T).reshape(t, kv_heads, head_dim)
            v = (h @ w["v"].T).reshape(t, kv_heads, head_dim)
            out = np.zeros((t, heads, head_dim))
            for head in range(heads):
                scores = q[:, head] @ k[:, 0].T / math.sqrt(head_dim)
                distance = np.arange(t)[None, :] - np.arange(t)[:, None]  # j - p
                scores = scores + 0.5 ** (head + 1) * distance
                scores = np.where(distance > 0, -np.inf, scores)
                probs = np.exp(scores - scores.max(axis=-1, keepdims=True))
                out[:, head] = (probs / probs.sum(axis=-1, keepdims=True)) @ v[:, 0]
            return out.reshape(t, heads * head_dim) @ w["o"].T

        def plain(tokens):
            eps = cfg["rms_norm_eps"]
            r = pl.embedding(weights["model.embed_tokens.weight"], np.array(tokens))
            cos, sin = pl.rope_tables(np.arange(len(tokens)), pl.config_inv_freq(cfg))
            for layer in range(2):
                q = f"model.layers.{layer}."
                h = pl.rms_norm(r, weights[q + "input_layernorm.weight"], eps)
                if layer == 0:
                    a, _ = pl.attention_layer(h, *(weights[q + f"self_attn.{n}_proj.weight"] for n in "qkvo"),
                                              cos, sin, heads, kv_heads, head_dim)
                else:
                    a = penalized_attention(h, q)
                r = r + a
                r = r + pl.swiglu(pl.rms_norm(r, weights[q + "post_attention_layernorm.weight"], eps),
                                  *(weights[q + f"mlp.{n}_proj.weight"] for n in ("gate", "up", "down")))
            return pl.rms_norm(r, weights["model.norm.weight"], eps) @ weights["lm_head.weight"].astype(np.float64).T

        requests = {f"d{i}": tiny.random_tokens(cfg, n, seed=30 + i) for i, n in enumerate((70, 9, 33))}
        expected = {rid: plain(t) for rid, t in requests.items()}
        # the penalty matters: without it (and without rotation) layer 1 gives other logits
        runner = ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=24, block_size=16, max_concurrent=3)
        groups = runner.cache.groups
        if dtype == "bfloat16":
            assert [g.v_transposed for g in groups] == [True, False] and [g.calls for g in groups] == [[0], [1]]
        else:
            assert len(groups) == 1 and not groups[0].v_transposed
        got = ru.run_schedule(runner, requests, ru.schedule_mixed(requests, seed=7, tail=5))
        for rid in requests:
            ru.assert_close(got[rid], expected[rid], dtype, f"penalty {rid}")
        runner.cache.check()
    finally:
        ARCHITECTURES.unregister("ToyPenaltyTestLM")
        POSITION_ENCODINGS.unregister("distance_penalty")


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_mixer_with_keys_and_values_of_different_widths(tmp_path, dtype):
    """A paged mixer defined here keeps narrow keys (8 per token) and wide values (24): it
    declares both widths, the cache manager sizes the two streams apart and hands the
    mixer pages of each, and the mixer reads and writes them through the step's block
    tables and write slots.  No framework file knows it."""
    import copy
    import dataclasses

    from mini_infer_amd.engine import ModelRunner
    from mini_infer_amd.models.spec import LayerSpec
    from mini_infer_amd.parts import CacheNeeds, Mixer, PagedKVNeeds, ParamSpec
    from mini_infer_amd.registry import ARCHITECTURES, MIXERS

    hidden, k_dim, v_dim = tiny.TINY_A["hidden_size"], 8, 24

    class NarrowKeysWideValues(Mixer):
        def param_specs(self, prefix):
            return {prefix + "k.weight": ParamSpec((k_dim, hidden)), prefix + "q.weight": ParamSpec((k_dim, hidden)),
                    prefix + "v.weight": ParamSpec((v_dim, hidden)), prefix + "o.weight": ParamSpec((hidden, v_dim))}

        def load_params(self, prefix, get):
            self.w = {n: get(prefix + n + ".weight").float() for n in "qkvo"}

        def cache_needs(self, page_size):
            return CacheNeeds(pages=PagedKVNeeds(1, k_dim, v_head_dim=v_dim))

        def forward(self, x, ctx, cache, writes_cache=True):
            page = ctx.page_size
            assert cache.k_pages.shape[1:] == (1, page, k_dim) and cache.v_pages.shape[1:] == (1, page, v_dim)
            xf = x.float()
            q, k, v = xf @ self.w["q"].T, xf @ self.w["k"].T, xf @ self.w["v"].T
            slots = ctx.slot_mapping[cache.group].long()
            cache.k_pages[slots // page, 0, slots % page] = k.to(x.dtype)
            cache.v_pages[slots // page, 0, slots % page] = v.to(x.dtype)
            out = torch.empty((x.shape[0], v_dim), dtype=torch.float32, device=x.device)
            table = ctx.block_tables[cache.group]
            for b in range(ctx.num_requests):
                first, last = ctx.host_cu_seqlens_q[b], ctx.host_cu_seqlens_q[b + 1]
                length = ctx.host_seq_lens[b]
                pages = table[b, : -(-length // page)].long()
                keys = cache.k_pages[pages, 0].reshape(-1, k_dim)[:length].float()
                values = cache.v_pages[pages, 0].reshape(-1, v_dim)[:length].float()
                scores = q[first:last] @ keys.T
                positions = ctx.positions[first:last].long()
                hidden_keys = torch.arange(length, device=x.device)[None, :] > positions[:, None]
                out[first:last] = torch.softmax(scores.masked_fill(hidden_keys, float("-inf")), dim=-1) @ values
            return (out @ self.w["o"].T).to(x.dtype)

    MIXERS.register("narrow_keys_wide_values", lambda desc, dtype_, device, shared=None: NarrowKeysWideValues(dtype_, device))

    def with_toy(spec):
        layers = list(spec.layers)
        block = copy.deepcopy(layers[0].block)
        block["mixer"] = {"kind": "narrow_keys_wide_values"}
        layers[0] = LayerSpec(layers[0].prefix, block)
        return dataclasses.replace(spec, layers=layers)

    _register_variant("ToyWidthsTestLM", with_toy)
    try:
        cfg = dict(tiny.TINY_A, architectures=["ToyWidthsTestLM"])
        weights = tiny.make_weights(cfg, 66)
        for n in "qkvo":
            del weights[f"model.layers.0.self_attn.{n}_proj.weight"]
        rng = np.random.default_rng(8)
        p = "model.layers.0.self_attn."
        for n, shape in (("q", (k_dim, hidden)), ("k", (k_dim, hidden)), ("v", (v_dim, hidden)), ("o", (hidden, v_dim))):
            weights[p + n + ".weight"] = tiny.bf16_round(rng.standard_normal(shape) / math.sqrt(shape[1]))
        folder = tiny.write_model_dir(tmp_path / "widths", cfg, weights)
        rounded = (lambda a: tiny.bf16_round(a).astype(np.float64)) if dtype == "bfloat16" else (lambda a: a)

        def plain(tokens):
            eps = cfg["rms_norm_eps"]
            t = len(tokens)
            r = pl.embedding(weights["model.embed_tokens.weight"], np.array(tokens))
            h = rounded(pl.rms_norm(r, weights["model.layers.0.input_layernorm.weight"], eps))
            w = {n: weights[p + n + ".weight"].astype(np.float64) for n in "qkvo"}
            q, k, v = h @ w["q"].T, rounded(h @ w["k"].T), rounded(h @ w["v"].T)
            scores = np.where(np.arange(t)[None, :] > np.arange(t)[:, None], -np.inf, q @ k.T)
            probs = np.exp(scores - scores.max(axis=-1, keepdims=True))
            r = r + rounded(((probs / probs.sum(axis=-1, keepdims=True)) @ v) @ w["o"].T)
            q0 = "model.layers.0."
            r = r + pl.swiglu(pl.rms_norm(r, weights[q0 + "post_attention_layernorm.weight"], eps),
                              *(weights[q0 + f"mlp.{n}_proj.weight"] for n in ("gate", "up", "down")))
            q1 = "model.layers.1."
            cos, sin = pl.rope_tables(np.arange(t), pl.config_inv_freq(cfg))
            a, _ = pl.attention_layer(pl.rms_norm(r, weights[q1 + "input_layernorm.weight"], eps),
                                      *(weights[q1 + f"self_attn.{n}_proj.weight"] for n in "qkvo"), cos, sin, 4, 2, 16)
            r = r + a
            r = r + pl.swiglu(pl.rms_norm(r, weights[q1 + "post_attention_layernorm.weight"], eps),
                              *(weights[q1 + f"mlp.{n}_proj.weight"] for n in ("gate", "up", "down")))
            return pl.rms_norm(r, weights["model.norm.weight"], eps) @ weights["model.embed_tokens.weight"].astype(np.float64).T

        requests = {f"w{i}": tiny.random_tokens(cfg, n, seed=40 + i) for i, n in enumerate((19, 8, 27, 12))}
        expected = {rid: plain(t) for rid, t in requests.items()}
        runner = ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=20, block_size=4, max_concurrent=4)
        groups = runner.cache.groups
        assert [(g.head_dim, g.value_dim) for g in groups] == [(k_dim, v_dim), (16, 16)]
        assert groups[0].k_storage.shape[-1] == 4 * k_dim and groups[0].v_storage.shape[-1] == 4 * v_dim
        got = ru.run_schedule(runner, requests, ru.schedule_mixed(requests, seed=8, tail=4))
        for rid in requests:
            ru.assert_close(got[rid], expected[rid], dtype, f"widths {rid}")
        runner.cache.check()
        assert all(g.pool.num_free == 20 for g in groups)
    finally:
        ARCHITECTURES.unregister("ToyWidthsTestLM")
        MIXERS.unregister("narrow_keys_wide_values")


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_embedding_and_head_register_and_take_the_places_of_the_built_in_ones(tmp_path, dtype):
    """How the residual stream starts and ends is a part like any other: an embedding defined
    here adds a learned row per position to the token's row, and a head defined here caps the
    logits with a tanh.  The model's spec names them by kind; no framework file changes."""
    import dataclasses

    from mini_infer_amd import ops
    from mini_infer_amd.engine import ModelRunner
    from mini_infer_amd.parts import Embedding, Head, ParamSpec
    from mini_infer_amd.registry import ARCHITECTURES, EMBEDDINGS, HEADS

    cfg = dict(tiny.TINY_A, architectures=["ToyEndsTestLM"], max_position_embeddings=64)
    hidden, vocab, cap = cfg["hidden_size"], cfg["vocab_size"], 100.0

    class TokensPlusPositions(Embedding):
        def param_specs(self, prefix):
            return {"model.embed_tokens.weight": ParamSpec((vocab, hidden)),
                    "model.embed_positions.weight": ParamSpec((64, hidden))}

        def load_params(self, prefix, get):
            self.weight = get("model.embed_tokens.weight").contiguous()
            self.rows = get("model.embed_positions.weight").contiguous()

        def forward(self, ctx):
            return ops.embed_gather(self.weight, ctx.token_ids) + ops.embed_gather(self.rows, ctx.positions)

    class CappedHead(Head):
        def __init__(self, dtype_, device, embedding):
            super().__init__(dtype_, device)
            self.embedding = embedding

        def forward(self, h, ctx):
            return cap * torch.tanh(ops.linear(h, self.embedding.weight).float() / cap)

    EMBEDDINGS.register("tokens_plus_positions", lambda desc, dtype_, device, shared=None: TokensPlusPositions(dtype_, device))
    HEADS.register("capped_head", lambda desc, dtype_, device, shared=None: CappedHead(dtype_, device, shared["embedding"]))
    _register_variant("ToyEndsTestLM", lambda spec: dataclasses.replace(
        spec, embedding={"kind": "tokens_plus_positions"}, head={"kind": "capped_head"}))
    try:
        weights = tiny.make_weights(cfg, 67)
        weights["model.embed_positions.weight"] = tiny.bf16_round(np.random.default_rng(9).standard_normal((64, hidden)))
        folder = tiny.write_model_dir(tmp_path / "ends", cfg, weights)

        def plain(tokens):
            eps = cfg["rms_norm_eps"]
            r = pl.embedding(weights["model.embed_tokens.weight"], np.array(tokens))
            r = r + weights["model.embed_positions.weight"][: len(tokens)].astype(np.float64)
            cos, sin = pl.rope_tables(np.arange(len(tokens)), pl.config_inv_freq(cfg))
            for layer in range(2):
                q = f"model.layers.{layer}."
                a, _ = pl.attention_layer(
                    pl.rms_norm(r, weights[q + "input_layernorm.weight"], eps),
                    *(weights[q + f"self_attn.{n}_proj.weight"] for n in "qkvo"), cos, sin, 4, 2, 16)
                r = r + a
                r = r + pl.swiglu(pl.rms_norm(r, weights[q + "post_attention_layernorm.weight"], eps),
                                  *(weights[q + f"mlp.{n}_proj.weight"] for n in ("gate", "up", "down")))
            logits = pl.rms_norm(r, weights["model.norm.weight"], eps) @ weights["model.embed_tokens.weight"].astype(np.float64).T
            return cap * np.tanh(logits / cap)

        requests = {f"e{i}": tiny.random_tokens(cfg, n, seed=50 + i) for i, n in enumerate((21, 5, 14))}
        expected = {rid: plain(t) for rid, t in requests.items()}
        assert np.abs(expected["e0"] - pl.llama_logits(cfg, weights, np.array(requests["e0"]))).max() > 1e-1
        runner = ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=24, block_size=4, max_concurrent=3)
        got = ru.run_schedule(runner, requests, ru.schedule_mixed(requests, seed=9, tail=5))
        for rid in requests:
            ru.assert_close(got[rid], expected[rid], dtype, f"ends {rid}")
    finally:
        ARCHITECTURES.unregister("ToyEndsTestLM")
        EMBEDDINGS.unregister("tokens_plus_positions")
        HEADS.unregister("capped_head")


_LONG = {}


def _long_case():
    """8,300 tokens of tiny B and their plain logits (made once, by the plain model's torch twin in
    float64 on the GPU: the NumPy one takes half a minute at this length)."""
    if not _LONG:
        import plain_llama_torch as plt

        cfg = dict(tiny.TINY_B, max_position_embeddings=16384)
        weights = tiny.make_weights(cfg, 57)
        tokens = tiny.random_tokens(cfg, 8300, seed=12)
        expected = ru.Oracle(plt.llama_logits(cfg, weights, tokens, device=DEV),
                             plt.llama_logits(cfg, weights, tokens, device=DEV, store=plt.bf16_round))
        _LONG.update(cfg=cfg, weights=weights, tokens=tokens, expected=expected)
    return _LONG


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_block_arrangement_and_toy_norm_in_one_layer_of_two(tmp_path, dtype):
    """Layer 0 is Llama's; layer 1 is described with a block kind and a norm kind defined here:
    ONE norm (centred, with a bias: mean and variance instead of the mean square) whose output
    feeds the attention and the feed-forward side by side, their sum going to the residual.  The
    model is built layer by layer from the descriptions, loaded by tensor name (the toy norm's
    bias included), stepped in portions and as recorded single tokens: no framework file changes."""
    import copy
    import dataclasses

    from mini_infer_amd.engine import ModelRunner
    from mini_infer_amd.models.spec import LayerSpec
    from mini_infer_amd.parts import Block, Norm, ParamSpec
    from mini_infer_amd.registry import ARCHITECTURES, BLOCKS, FEED_FORWARDS, MIXERS, NORMS

    hidden = tiny.TINY_A["hidden_size"]
    toy_eps = 3e-4

    class CentredNorm(Norm):
        graph_safe = True

        def param_specs(self, prefix):
            return {prefix + "weight": ParamSpec((hidden,), init="norm_weight"), prefix + "bias": ParamSpec((hidden,))}

        def load_params(self, prefix, get):
            self.weight, self.bias = get(prefix + "weight").float(), get(prefix + "bias").float()

        def forward(self, delta, residual, rows=None):
            if delta is not None:
                residual += delta.float()
            centred = residual - residual.mean(dim=-1, keepdim=True)
            variance = (centred * centred).mean(dim=-1, keepdim=True)
            return (centred * torch.rsqrt(variance + toy_eps) * self.weight + self.bias).to(self.dtype)

    class SideBySide(Block):
        def __init__(self, norm, mixer, feed_forward, dtype_, device):
            super().__init__(dtype_, device)
            self.norm, self.mixer, self.feed_forward = norm, mixer, feed_forward

        @property
        def graph_safe(self):
            return self.norm.graph_safe and self.mixer.graph_safe and self.feed_forward.graph_safe

        def _children(self):
            return (("input_layernorm.", self.norm), ("self_attn.", self.mixer), ("mlp.", self.feed_forward))

        def param_specs(self, prefix):
            specs = {}
            for sub, part in self._children():
                specs.update(part.param_specs(prefix + sub))
            return specs

        def load_params(self, prefix, get):
            for sub, part in self._children():
                part.load_params(prefix + sub, get)

        def forward(self, delta, residual, ctx, cache, writes_cache=True):
            h = self.norm.forward(delta, residual)
            return self.mixer.forward(h, ctx, cache, writes_cache) + self.feed_forward.forward(h, ctx)

    NORMS.register("centred_norm", lambda desc, dtype_, device, shared=None: CentredNorm(dtype_, device))
    BLOCKS.register(
        "side_by_side",
        lambda desc, dtype_, device, shared=None: SideBySide(
            NORMS.lookup(desc["norm"]["kind"])(desc["norm"], dtype_, device, shared),
            MIXERS.lookup(desc["mixer"]["kind"])(desc["mixer"], dtype_, device, shared),
            FEED_FORWARDS.lookup(desc["feed_forward"]["kind"])(desc["feed_forward"], dtype_, device, shared),
            dtype_, device,
        ),
    )

    def with_toy(spec):
        layers = list(spec.layers)
        block = copy.deepcopy(layers[1].block)
        block["kind"] = "side_by_side"
        block["norm"] = {"kind": "centred_norm"}
        layers[1] = LayerSpec(layers[1].prefix, block)
        return dataclasses.replace(spec, layers=layers)

    _register_variant("ToyBlockTestLM", with_toy)
    try:
        cfg = dict(tiny.TINY_A, architectures=["ToyBlockTestLM"])
        weights = tiny.make_weights(cfg, 64)
        del weights["model.layers.1.post_attention_layernorm.weight"]
        rng = np.random.default_rng(6)
        weights["model.layers.1.input_layernorm.bias"] = tiny.bf16_round(rng.standard_normal(hidden) / 4)
        folder = tiny.write_model_dir(tmp_path / "toy", cfg, weights)

        def plain(tokens):
            eps = cfg["rms_norm_eps"]
            w = {k: v.astype(np.float64) for k, v in weights.items()}
            r = pl.embedding(weights["model.embed_tokens.weight"], np.array(tokens))
            cos, sin = pl.rope_tables(np.arange(len(tokens)), pl.config_inv_freq(cfg))
            p = "model.layers.0."
            a, _ = pl.attention_layer(pl.rms_norm(r, w[p + "input_layernorm.weight"], eps),
                                      *(w[p + f"self_attn.{n}_proj.weight"] for n in "qkvo"), cos, sin, 4, 2, 16)
            r = r + a
            r = r + pl.swiglu(pl.rms_norm(r, w[p + "post_attention_layernorm.weight"], eps),
                              *(w[p + f"mlp.{n}_proj.weight"] for n in ("gate", "up", "down")))
            p = "model.layers.1."
            centred = r - r.mean(axis=-1, keepdims=True)
            h = centred / np.sqrt((centred * centred).mean(axis=-1, keepdims=True) + toy_eps)
            h = h * w[p + "input_layernorm.weight"] + w[p + "input_layernorm.bias"]
            if dtype == "bfloat16":
                h = tiny.bf16_round(h).astype(np.float64)
            a, _ = pl.attention_layer(h, *(w[p + f"self_attn.{n}_proj.weight"] for n in "qkvo"), cos, sin, 4, 2, 16)
            r = r + a + pl.swiglu(h, *(w[p + f"mlp.{n}_proj.weight"] for n in ("gate", "up", "down")))
            return pl.rms_norm(r, w["model.norm.weight"], eps) @ w["model.embed_tokens.weight"].T

        requests = {f"s{i}": tiny.random_tokens(cfg, n, seed=40 + i) for i, n in enumerate((26, 11, 19))}
        expected = {rid: plain(t) for rid, t in requests.items()}
        runner = ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=24, block_size=4, max_concurrent=3)
        assert type(runner.model.blocks[1]).__name__ == "SideBySide" and type(runner.model.blocks[0]).__name__ == "PreNormBlock"
        assert runner.model.graph_safe and runner.decode_graphs is not None
        got = ru.run_schedule(runner, requests, ru.schedule_mixed(requests, seed=8, max_live=3, tail=6))
        for rid in requests:
            ru.assert_close(got[rid], expected[rid], dtype, f"toy block {rid}")
        assert runner.decode_graphs.replays > 0
        runner.cache.check()
        assert runner.num_free_blocks() == 24
    finally:
        ARCHITECTURES.unregister("ToyBlockTestLM")
        BLOCKS.unregister("side_by_side")
        NORMS.unregister("centred_norm")


def test_a_whole_architecture_with_config_keys_and_tensor_names_of_its_own(tmp_path):
    """An architecture defined here from nothing but the framework's parts: config.json keys of
    its own (read into a typed configuration of its own, which refuses what it does not know),
    tensor names of its own, a feed-forward of another width in each layer, the layers run
    twice over.  Registered under its name it gets a model folder with random weights from
    the random-weights mode, is loaded by tensor name, steps and generates through `LLM` as
    Llama does; the plain functions, fed the renamed tensors layer by layer, give the same
    logits and the same greedy tokens.  No framework file changes."""
    import dataclasses
    import json

    from safetensors.torch import load_file

    from mini_infer_amd.engine import StepEntry
    from mini_infer_amd.engine.llm import LLM
    from mini_infer_amd.models.spec import Architecture, LayerCall, LayerSpec, ModelSpec
    from mini_infer_amd.registry import ARCHITECTURES
    from mini_infer_amd.weights import write_random_model

    @dataclasses.dataclass(frozen=True)
    class ToyConfig:
        n_layer: int
        d_model: int
        n_head: int
        n_kv_head: int
        d_head: int
        d_ff: tuple
        n_vocab: int
        norm_eps: float
        rope_base: float
        loops: int

        @classmethod
        def from_dict(cls, raw):
            unknown = set(raw) - {f.name for f in dataclasses.fields(cls)} - {"architectures"}
            if unknown:
                raise ValueError(f"unknown keys in a TinyToyLM config: {sorted(unknown)}")
            if len(raw["d_ff"]) != raw["n_layer"]:
                raise ValueError("d_ff lists one width per layer")
            return cls(**{k: (tuple(v) if k == "d_ff" else v) for k, v in raw.items() if k != "architectures"})

    def toy_spec(cfg):
        norm = {"kind": "rms_norm", "hidden_size": cfg.d_model, "eps": cfg.norm_eps}
        layers = [
            LayerSpec(prefix=f"blocks.{i}.", block={
                "kind": "pre_norm",
                "norm": norm,
                "mixer": {"kind": "gqa_attention", "hidden_size": cfg.d_model, "num_heads": cfg.n_head,
                          "num_kv_heads": cfg.n_kv_head, "head_dim": cfg.d_head,
                          "position": {"kind": "rotary", "head_dim": cfg.d_head, "theta": cfg.rope_base}},
                "feed_forward": {"kind": "swiglu", "hidden_size": cfg.d_model, "intermediate_size": cfg.d_ff[i]},
                "names": {"mixer_norm": "ln1.", "mixer": "attn.", "ffn_norm": "ln2.", "feed_forward": "ff."},
            })
            for i in range(cfg.n_layer)
        ]
        return ModelSpec(
            vocab_size=cfg.n_vocab, hidden_size=cfg.d_model, embedding_name="wte.weight", layers=layers,
            order=[LayerCall(i) for _ in range(cfg.loops) for i in range(cfg.n_layer)],
            final_norm=norm, final_norm_prefix="ln_f.", tie_word_embeddings=True,
        )

    raw = {"architectures": ["TinyToyLM"], "n_layer": 2, "d_model": 96, "n_head": 6, "n_kv_head": 3, "d_head": 16,
           "d_ff": [80, 208], "n_vocab": 211, "norm_eps": 2e-5, "rope_base": 7000.0, "loops": 2}
    ARCHITECTURES.register("TinyToyLM", Architecture("TinyToyLM", ToyConfig.from_dict, toy_spec))
    try:
        with pytest.raises(ValueError, match="unknown keys"):
            ToyConfig.from_dict(dict(raw, hidden_size=5))
        folder = write_random_model(raw, seed=11, out_dir=tmp_path / "toy_arch", std=0.25, norm_jitter=0.2)
        assert json.loads((folder / "config.json").read_text()) == raw
        weights = {k: v.double().numpy() for k, v in load_file(str(folder / "model.safetensors")).items()}
        assert sorted(weights)[:3] == ["blocks.0.attn.k_proj.weight", "blocks.0.attn.o_proj.weight", "blocks.0.attn.q_proj.weight"]
        assert "wte.weight" in weights and "ln_f.weight" in weights and len(weights) == 2 * 9 + 2
        assert weights["blocks.0.ff.gate_proj.weight"].shape == (80, 96) and weights["blocks.1.ff.gate_proj.weight"].shape == (208, 96)

        # the plain Llama model under Llama's names: the same formulas, the toy's tensors and order
        renamed = {"model.embed_tokens.weight": weights["wte.weight"], "model.norm.weight": weights["ln_f.weight"]}
        for i in range(2):
            for ours, llamas in (("ln1.", "input_layernorm."), ("ln2.", "post_attention_layernorm."),
                                 *((f"attn.{n}_proj.", f"self_attn.{n}_proj.") for n in "qkvo"),
                                 *((f"ff.{n}_proj.", f"mlp.{n}_proj.") for n in ("gate", "up", "down"))):
                renamed[f"model.layers.{i}.{llamas}weight"] = weights[f"blocks.{i}.{ours}weight"]
        as_llama = {"num_hidden_layers": 2, "hidden_size": 96, "num_attention_heads": 6, "num_key_value_heads": 3,
                    "head_dim": 16, "rms_norm_eps": 2e-5, "rope_theta": 7000.0, "tie_word_embeddings": True}
        looped = [(0, None), (1, None), (0, None), (1, None)]

        def plain(tokens):
            return pl.llama_logits(as_llama, renamed, np.array(tokens), order=looped)

        llm = LLM(folder, dtype="float32", num_blocks=48, block_size=4, max_num_batched_tokens=16, chunk_size=16)
        assert len(llm.runner.cache.layer_caches()) == 4  # two layers, each called twice, each call with its own cache
        rng = np.random.default_rng(12)
        prompts = [[int(t) for t in rng.integers(0, 211, size=n)] for n in (9, 23, 1)]
        for prompt, result in zip(prompts, llm.generate(prompts, max_tokens=6)):
            tokens = list(prompt)
            for _ in range(6):
                tokens.append(pl.greedy(plain(tokens)[-1]))
            assert result.tokens == tokens[len(prompt):]
        # the step function on a whole prompt: the logits, not only their maxima
        logits = llm.runner.step([StepEntry("whole", prompts[1], list(range(23)))]).cpu().numpy()
        llm.runner.free_request("whole")
        ru.assert_close(logits, plain(prompts[1]), "float32", "toy architecture, whole prompt")
        assert llm.runner.num_free_blocks() == 48
        # and in bfloat16, a portion and then single tokens (widths of 80 and 208: not every kernel's sizes)
        from mini_infer_amd.engine import ModelRunner

        runner = ModelRunner.from_pretrained(folder, dtype="bfloat16", num_blocks=8, block_size=4)
        got = [runner.step([StepEntry("b", prompts[1][:17], list(range(17)))]).cpu().numpy()]
        got += [runner.step([StepEntry("b", [t], [0])]).cpu().numpy() for t in prompts[1][17:]]
        ru.assert_close(np.concatenate(got), ru.oracle(as_llama, renamed, prompts[1], order=looped), "bfloat16",
                        "toy architecture, bfloat16")
        assert runner.decode_graphs.replays == 6
    finally:
        ARCHITECTURES.unregister("TinyToyLM")


def test_an_architecture_of_another_overall_shape_brings_a_model_object_of_its_own(tmp_path):
    """Not embedding -> blocks -> one norm -> one head: a model with two heads whose logits are
    added, built by the architecture's own `build_model` from the package's parts.  Loader,
    random-weights mode, runner, scheduler and `LLM` work from the model contract alone."""
    import dataclasses

    from safetensors.torch import load_file

    from mini_infer_amd.engine.llm import LLM
    from mini_infer_amd.models.spec import Architecture
    from mini_infer_amd.parts.embedding import OutputHead, TokenEmbedding
    from mini_infer_amd.parts.norm import RMSNorm
    from mini_infer_amd.registry import ARCHITECTURES
    from mini_infer_amd.weights import write_random_model

    @dataclasses.dataclass(frozen=True)
    class TwoHeadConfig:
        width: int
        vocab: int
        eps: float

        @classmethod
        def from_dict(cls, raw):
            return cls(int(raw["width"]), int(raw["vocab"]), float(raw["eps"]))

    class TwoHeadModel:
        graph_safe = True
        max_position_embeddings = None

        def __init__(self, config, dtype, device):
            self.dtype, self.device, self.vocab_size = dtype, torch.device(device), config.vocab
            self.embedding = TokenEmbedding(config.vocab, config.width, "table", dtype, device)
            self.norm = RMSNorm(config.width, config.eps, dtype, device)
            self.heads = [OutputHead(config.width, config.vocab, f"head_{n}", dtype, device) for n in "ab"]

        def param_specs(self):
            specs = {**self.embedding.param_specs(""), **self.norm.param_specs("norm.")}
            for head in self.heads:
                specs.update(head.param_specs(""))
            return specs

        def optional_names(self):
            return set()

        def load_params(self, get):
            self.embedding.load_params("", get)
            self.norm.load_params("norm.", get)
            for head in self.heads:
                head.load_params("", get)

        def cache_needs(self, page_size):
            return []

        def forward(self, ctx, caches):
            h = self.norm.forward(None, self.embedding.forward(ctx), rows=ctx.logit_rows)
            return self.heads[0].forward(h, ctx) + self.heads[1].forward(h, ctx)

    raw = {"architectures": ["TwoHeadTestLM"], "width": 64, "vocab": 97, "eps": 1e-5}
    ARCHITECTURES.register("TwoHeadTestLM", Architecture("TwoHeadTestLM", TwoHeadConfig.from_dict, build_model=TwoHeadModel))
    try:
        with pytest.raises(ValueError, match="one of the two"):
            Architecture("Neither", TwoHeadConfig.from_dict)
        folder = write_random_model(raw, seed=3, out_dir=tmp_path / "two_heads", std=0.5, norm_jitter=0.2, dtype="float32")
        weights = {k: v.double().numpy() for k, v in load_file(str(folder / "model.safetensors")).items()}
        assert sorted(weights) == ["head_a", "head_b", "norm.weight", "table"]

        def plain_next(token):
            h = pl.rms_norm(weights["table"][[token]], weights["norm.weight"], raw["eps"])
            return int(np.argmax(h @ (weights["head_a"] + weights["head_b"]).T))

        llm = LLM(folder, dtype="float32", num_blocks=1, block_size=4, max_concurrent=2)
        assert not llm.runner.cache.has_pages and not llm.runner.cache.states.has_state
        prompts = [[5, 9, 33], [96], [1, 2]]
        for prompt, result in zip(prompts, llm.generate(prompts, max_tokens=5)):
            expected, last = [], prompt[-1]
            for _ in range(5):
                last = plain_next(last)
                expected.append(last)
            assert result.tokens == expected and result.finish_reason == "length"
        assert llm.runner.decode_graphs.replays > 0
    finally:
        ARCHITECTURES.unregister("TwoHeadTestLM")


@pytest.mark.parametrize("dtype", DTYPES)
def test_context_past_eight_thousand_keys(tmp_path, dtype):
    """8,288 tokens in portions of 2,048, then 12 tokens one by one, where single tokens'
    keys are cut into the many ranges of long contexts.  (In float32 a page read from the
    wrong place anywhere in the 8,000 moves the logits by far more than the tolerance; for
    bfloat16 the kernel tests plant single far keys.)"""
    from mini_infer_amd.engine import ModelRunner, StepEntry

    case = _long_case()
    tokens, expected = case["tokens"], case["expected"]
    folder = tiny.write_model_dir(tmp_path / "long", case["cfg"], case["weights"])
    runner = ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=len(tokens) // 16 + 2, block_size=16)
    got, fed, whole = [], 0, len(tokens) - 12
    while fed < whole:
        count = min(2048, whole - fed)
        want = list(range(count - 5, count))  # the last five places of each portion
        got.append((fed + count - 5, runner.step([StepEntry("r", tokens[fed : fed + count], want)]).cpu().numpy()))
        fed += count
    for _ in range(12):
        got.append((fed, runner.step([StepEntry("r", tokens[fed : fed + 1], [0])]).cpu().numpy()))
        fed += 1
    places = [start + i for start, rows in got for i in range(len(rows))]
    ru.assert_close(np.concatenate([rows for _, rows in got]), expected[places], dtype, "long context")
    runner.free_request("r")
    runner.cache.check()


def test_products_left_in_partial_sums_through_the_engine(tmp_path, monkeypatch):
    """The tiny models never meet the sizes at which a product is left as sums over ranges of
    K for the next norm; here the rule is made to say yes always, so that every o and down
    product of a replay (portions, single tokens, mixed batches up to 64 rows) takes that way."""
    from mini_infer_amd.engine import ModelRunner
    from mini_infer_amd.ops import kernels

    taken = []

    def always(m, n, k):
        taken.append((m, n, k))
        return m <= kernels.PARTIAL_SUMS_MAX_ROWS

    monkeypatch.setattr(kernels, "partial_sums_pay", always)
    cfg, block, weights, folder = _folder(tmp_path, "B", 58)
    requests = {f"p{i}": tiny.random_tokens(cfg, n, seed=30 + i) for i, n in enumerate((70, 33, 90, 41, 57))}
    expected = {rid: ru.oracle(cfg, weights, t) for rid, t in requests.items()}
    runner = ModelRunner.from_pretrained(folder, dtype="bfloat16", num_blocks=20, block_size=block, max_concurrent=4)
    for schedule in (ru.schedule_prefill_then_decode(requests, tail=8), ru.schedule_mixed(requests, seed=7, tail=6)):
        got = ru.run_schedule(runner, requests, schedule)
        for rid in requests:
            ru.assert_close(got[rid], expected[rid], "bfloat16", f"partial sums {rid}")
    rows = {m for m, _, _ in taken}
    assert 1 in rows and any(m > 16 for m in rows) and len({(n, k) for _, n, k in taken}) == 2  # o and down
    runner.cache.check()
