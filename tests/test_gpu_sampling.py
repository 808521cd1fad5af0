"""The sampling kernel against the plain filters and distribution."""

import numpy as np
import pytest
import torch

import plain_llama as pl

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _sample(logits, params, seeds, draws):
    from mini_infer_amd.sampling import sample_batch

    return sample_batch(logits.to(DEV), params, seeds, draws)


def _params(**kw):
    from mini_infer_amd.sampling import SamplingParams

    return SamplingParams(**kw)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_greedy_is_first_maximum(dtype):
    logits = torch.tensor([[1.0, 5.0, 3.0, 2.0], [7.0, -1.0, 7.0, 7.0], [-3.0, -2.0, -2.0, -9.0]]).to(dtype)
    assert _sample(logits, [_params()] * 3, [0] * 3, [0] * 3) == [1, 0, 1]
    big = torch.randn(5, 128256, generator=torch.Generator().manual_seed(0)).to(dtype)
    big[2, 77777] = 50.0
    big[3, 128255] = 50.0
    big[4, 5] = big[4, 100000] = 60.0
    got = _sample(big, [_params()] * 5, [0] * 5, [0] * 5)
    assert got == big.float().argmax(dim=-1).tolist()[:2] + [77777, 128255, 5]


def test_top_k_one_and_tiny_top_p_are_greedy():
    logits = torch.randn(4, 1000, generator=torch.Generator().manual_seed(1))
    expected = logits.argmax(dim=-1).tolist()
    assert _sample(logits, [_params(temperature=10.0, top_k=1)] * 4, [1, 2, 3, 4], [0] * 4) == expected
    assert _sample(logits, [_params(temperature=1.0, top_p=0.001)] * 4, [1, 2, 3, 4], [0] * 4) == expected
    assert _sample(logits, [_params(temperature=1.0, top_p=0.0)] * 4, [1, 2, 3, 4], [0] * 4) == expected


def test_same_seed_same_tokens_whatever_the_batch():
    logits = torch.randn(6, 5000, generator=torch.Generator().manual_seed(2))
    params = [_params(temperature=0.8)] * 6
    seeds = [11, 12, 13, 14, 15, 2**63 + 5]
    draws = [0, 1, 2, 3, 4, 5]
    together = _sample(logits, params, seeds, draws)
    assert together == _sample(logits, params, seeds, draws)
    for i in range(6):
        assert _sample(logits[i : i + 1], params[:1], seeds[i : i + 1], draws[i : i + 1]) == [together[i]]
    rev = list(range(5, -1, -1))
    assert _sample(logits[rev], params, [seeds[i] for i in rev], [draws[i] for i in rev]) == [together[i] for i in rev]
    # another seed or another draw index gives other tokens somewhere
    assert _sample(logits, params, [s + 1 for s in seeds], draws) != together
    assert _sample(logits, params, seeds, [d + 1 for d in draws]) != together
    # greedy rows in the same batch are untouched by the sampled rows
    mixed = _sample(logits, [_params()] * 3 + [_params(temperature=0.8)] * 3, seeds, draws)
    assert mixed[:3] == logits[:3].argmax(dim=-1).tolist() and mixed[3:] == together[3:]


def _frequencies(logits_row, params, draws=20000):
    rows = logits_row.unsqueeze(0).repeat(draws, 1)
    got = _sample(rows, [params] * draws, [99] * draws, list(range(draws)))
    return np.bincount(got, minlength=logits_row.numel()) / draws


def test_draws_follow_the_softmax():
    logits = torch.tensor([0.0, float(np.log(3.0)), -1.0, 0.5], dtype=torch.float32)
    freq = _frequencies(logits, _params(temperature=1.0))
    expected = pl.sampling_distribution(logits.numpy(), 1.0)
    assert np.abs(freq - expected).max() < 0.012
    freq = _frequencies(logits, _params(temperature=0.5))
    assert np.abs(freq - pl.sampling_distribution(logits.numpy(), 0.5)).max() < 0.012


@pytest.mark.parametrize("top_k,top_p", [(3, 1.0), (0, 0.7), (5, 0.5), (2, 0.95), (0, 0.3)])
def test_filters_match_the_plain_filters(top_k, top_p):
    logits = torch.randn(40, generator=torch.Generator().manual_seed(3)) * 2.0
    freq = _frequencies(logits, _params(temperature=1.3, top_k=top_k, top_p=top_p), draws=12000)
    expected = pl.sampling_distribution(logits.numpy(), 1.3, top_k, top_p)
    assert set(np.nonzero(freq)[0]) <= set(np.nonzero(expected)[0]), "a filtered token was drawn"
    assert np.abs(freq - expected).max() < 0.02
    assert (freq[expected > 0.02] > 0).all()


def test_filters_on_a_large_vocabulary():
    """Thresholds found by radix descent equal thresholds found by sorting."""
    vocab = 128256
    logits = torch.randn(vocab, generator=torch.Generator().manual_seed(4)) * 3.0
    for top_k, top_p in ((50, 1.0), (0, 0.9), (1000, 0.6)):
        expected = pl.sampling_distribution(logits.numpy(), 0.9, top_k, top_p)
        allowed = set(np.nonzero(expected)[0])
        draws = 512
        rows = logits.unsqueeze(0).repeat(draws, 1)
        got = _sample(rows, [_params(temperature=0.9, top_k=top_k, top_p=top_p)] * draws, [5] * draws, list(range(draws)))
        assert set(got) <= allowed
        assert len(set(got)) > min(20, len(allowed) // 2)


def test_bad_arguments():
    from mini_infer_amd.sampling import SamplingParams, sample_tokens

    with pytest.raises(ValueError, match="temperature"):
        SamplingParams(temperature=-0.1)
    with pytest.raises(ValueError, match="top_k"):
        SamplingParams(top_k=-1)
    with pytest.raises(ValueError, match="top_p"):
        SamplingParams(top_p=1.5)
    with pytest.raises(ValueError, match="one params"):
        sample_tokens(torch.zeros(2, 4, device=DEV), [SamplingParams()], [0], [0])


def test_sampling_from_state_slots_is_sampling_with_the_same_settings_and_advances_the_draw():
    """Rows whose settings, seed and draw index are read from the requests' state slots give the
    tokens of the same settings handed over as arrays, draw after draw, with nothing sent
    from the host between the draws; slots not sampled are left alone."""
    from mini_infer_amd.cache import StateSlots
    from mini_infer_amd.sampling import sample_from_slots

    slots = StateSlots(6, {}, DEV)
    settings = [_params(temperature=0.8), _params(), _params(temperature=1.3, top_k=5),
                _params(temperature=0.6, top_p=0.8), _params(temperature=1.0, top_k=50, top_p=0.5)]
    seeds = [11, 12, 2**63 + 5, 14, 15]
    owned = [slots.allocate(f"r{i}") for i in range(6)]  # 5, 4, ... or any order: ids are what counts
    for slot, p, seed in zip(owned, settings, seeds):
        slots.set_sampling(slot, temperature=p.temperature, top_k=p.top_k, top_p=p.top_p, seed=seed, draw=0)
    order = [3, 0, 4, 1, 2]  # rows of the batch in another order than the slots
    row_slots = torch.tensor([owned[i] for i in order], dtype=torch.int32, device=DEV)
    for draw in range(4):
        logits = torch.randn(5, 3000, generator=torch.Generator().manual_seed(10 + draw)).to(DEV)
        expected = _sample(logits, [settings[i] for i in order], [seeds[i] for i in order], [draw] * 5)
        assert sample_from_slots(logits, row_slots, slots.table).tolist() == expected
    table = slots.table.cpu()
    assert [int(table[owned[i], 3]) for i in range(5)] == [4] * 5 and int(table[owned[5], 3]) == 0
    # one row alone, later: it goes on from its own draw index, whatever the others did
    logits = torch.randn(1, 3000, generator=torch.Generator().manual_seed(99)).to(DEV)
    alone = sample_from_slots(logits, row_slots[:1], slots.table).tolist()
    assert alone == _sample(logits, [settings[3]], [seeds[3]], [4])
    with pytest.raises(ValueError):
        sample_from_slots(logits, row_slots, slots.table)


def test_a_row_whose_slot_id_lies_outside_the_table_is_sampled_greedily_and_writes_nothing():
    """The padding rows of a recorded step carry slot -1: a caller that samples the whole bucket
    must not read or write memory before the table.  Such rows (and ids past the table's end)
    get the first largest logit, and the table is left as it was but for the real row's draw."""
    from mini_infer_amd.cache import StateSlots
    from mini_infer_amd.sampling import sample_from_slots

    slots = StateSlots(3, {}, DEV)
    real = slots.allocate("r")
    slots.set_sampling(real, temperature=0.9, top_k=0, top_p=1.0, seed=5, draw=2)
    before = slots.table.clone()
    logits = torch.randn(3, 777, generator=torch.Generator().manual_seed(3)).to(DEV)
    row_slots = torch.tensor([-1, real, 3], dtype=torch.int32, device=DEV)
    got = sample_from_slots(logits, row_slots, slots.table).tolist()
    assert got[0] == int(logits[0].argmax()) and got[2] == int(logits[2].argmax())
    assert got[1] == _sample(logits[1:2], [_params(temperature=0.9)], [5], [2])[0]
    after = slots.table.clone()
    assert int(after[real, 3]) == 3
    after[real, 3] = 2
    assert torch.equal(after, before)


def test_positions_and_draws_in_the_slot_table_follow_the_engine(tmp_path):
    """After steps of every kind (portions, recorded single-token steps, a request left out of a
    step) the device's slot table holds each request's length, as the host's copy does; a
    failed step leaves it as it was."""
    import tiny
    from mini_infer_amd.engine import ModelRunner, StepEntry
    from mini_infer_amd.exceptions import OutOfMemoryError

    cfg, block = tiny.CONFIGS["A"]
    folder = tiny.write_model_dir(tmp_path / "slots", cfg, tiny.make_weights(cfg, 70))
    runner = ModelRunner.from_pretrained(folder, dtype="bfloat16", num_blocks=12, block_size=block, max_concurrent=3)
    states = runner.cache.states

    def check():
        table = states.table.cpu().numpy()
        for rid in runner.cache.live_requests():
            slot = runner.cache.state_slot(rid)
            assert table[slot, 0] == runner.cache.length(rid) == states.position(slot), rid

    runner.step([StepEntry("a", tiny.random_tokens(cfg, 9, 1), [8]), StepEntry("b", tiny.random_tokens(cfg, 5, 2), [])])
    check()
    for step in range(6):  # recorded single-token steps of two requests, then of one
        entries = [StepEntry("a", [step + 1], [0])] + ([StepEntry("b", [step + 2], [0])] if step < 4 else [])
        runner.step(entries)
        assert runner.last_row_slots.tolist() == [runner.cache.state_slot(e.request_id) for e in entries]
        check()
    assert runner.decode_graphs.replays == 6
    with pytest.raises(OutOfMemoryError):
        runner.step([StepEntry("a", [1] * 40, [])])
    check()
    runner.free_request("b")
    runner.step([StepEntry("c", tiny.random_tokens(cfg, 7, 3), [6]), StepEntry("a", [3], [0])])
    assert runner.cache.state_slot("c") is not None
    check()
