"""The scheduler's decisions, with a model-free runner over the real cache manager (no GPU).

The fake runner's "logits" are a pure function of the tokens a request has fed so
far, so the tokens a request generates must not depend on batching, portions or
preemption; it also records every step so the tests can read the decisions.
"""

import numpy as np
import pytest
import torch

from mini_infer_amd.cache import CacheManager
from mini_infer_amd.engine.request import Request
from mini_infer_amd.engine.scheduler import ContinuousScheduler
from mini_infer_amd.exceptions import OutOfMemoryError
from mini_infer_amd.parts.base import CacheNeeds, PagedKVNeeds
from mini_infer_amd.sampling import SamplingParams

VOCAB = 50


def next_token(history: list[int]) -> int:
    return (sum(history) * 31 + 7 * len(history)) % VOCAB


class FakeRunner:
    def __init__(self, num_blocks=64, block_size=4, max_concurrent=8):
        self.num_blocks, self.block_size = num_blocks, block_size
        self.cache = CacheManager([CacheNeeds(pages=PagedKVNeeds(1, 16))], page_size=block_size,
                                  num_pages=num_blocks, max_requests=max_concurrent, allocate_storage=False)
        self.history: dict[int, list[int]] = {}
        self.steps: list[list[tuple[int, int, tuple]]] = []

    def num_free_blocks(self):
        return self.cache.num_free_pages()

    def step(self, entries):
        extents = {e.request_id: len(e.tokens) for e in entries}
        self.cache.reserve(extents)  # raises OutOfMemoryError with nothing changed
        rows = []
        for e in entries:
            if self.cache.length(e.request_id) == 0:
                self.history[e.request_id] = []
            assert len(self.history[e.request_id]) == self.cache.length(e.request_id)
            for i, token in enumerate(e.tokens):
                self.history[e.request_id].append(token)
                if i in e.want:
                    row = torch.zeros(VOCAB)
                    row[next_token(self.history[e.request_id])] = 1.0
                    rows.append(row)
        self.cache.commit(extents)
        self.cache.check()
        self.steps.append([(e.request_id, len(e.tokens), tuple(e.want)) for e in entries])
        return torch.stack(rows) if rows else torch.zeros((0, VOCAB))


def argmax_sampler(logits, params, seeds, draws):
    assert logits.shape[0] == len(params) == len(seeds) == len(draws)
    return logits.argmax(dim=-1).tolist()


def expected_tokens(prompt, count, eos=None):
    history, out = list(prompt), []
    for _ in range(count):
        token = next_token(history)
        if token == eos:
            break
        out.append(token)
        history.append(token)
    return out


def make(runner, **kwargs):
    kwargs.setdefault("sampler", argmax_sampler)
    return ContinuousScheduler(runner, **kwargs)


def prompt(n, seed):
    return np.random.default_rng(seed).integers(0, VOCAB, size=n).tolist()


def test_one_request_runs_to_length_and_frees_its_pages():
    runner = FakeRunner()
    sched = make(runner)
    result = sched.run(Request(prompt(10, 0), SamplingParams(), max_tokens=6))
    assert result.tokens == expected_tokens(prompt(10, 0), 6)
    assert result.finish_reason == "length" and result.prompt_tokens == 10
    assert runner.num_free_blocks() == runner.num_blocks
    # the prompt in one step, then one token a step; the last emitted token is never fed
    assert [s[0][1] for s in runner.steps] == [10, 1, 1, 1, 1, 1]
    assert len(runner.history[0]) == 10 + 5


def test_prompt_is_cut_by_chunk_size_and_logits_wanted_only_at_its_end():
    runner = FakeRunner()
    sched = make(runner, chunk_size=4)
    result = sched.run(Request(prompt(10, 1), SamplingParams(), max_tokens=2))
    assert [(n, want) for _, n, want in (s[0] for s in runner.steps)] == [(4, ()), (4, ()), (2, (1,)), (1, (0,))]
    assert result.tokens == expected_tokens(prompt(10, 1), 2)


def test_token_budget_decodes_first_then_portions_in_admission_order():
    runner = FakeRunner()
    sched = make(runner, chunk_size=100, max_num_batched_tokens=8)
    handles = [sched.submit(Request(prompt(n, n), SamplingParams(), max_tokens=4)) for n in (3, 9, 12)]
    while sched.step():
        pass
    for step in runner.steps:
        assert sum(n for _, n, _ in step) <= 8
    # step 0: request 0 whole (3), request 1 gets the remaining 5 of the budget
    assert runner.steps[0] == [(0, 3, (2,)), (1, 5, ())]
    # step 1: request 0 decodes first (1 token), then request 1's last 4, then 3 of request 2
    assert runner.steps[1] == [(0, 1, (0,)), (1, 4, (3,)), (2, 3, ())]
    assert any(n == 2 or n == 1 for s in runner.steps for _, n, _ in s)
    for handle, n in zip(handles, (3, 9, 12)):
        assert handle.wait().tokens == expected_tokens(prompt(n, n), 4)
    assert runner.num_free_blocks() == runner.num_blocks


def test_batched_equals_serial():
    prompts = [prompt(n, 10 + n) for n in (1, 5, 17, 30, 8)]
    serial = []
    for p in prompts:
        serial.append(make(FakeRunner()).run(Request(p, SamplingParams(), max_tokens=7)).tokens)
    runner = FakeRunner()
    sched = make(runner, chunk_size=6, max_num_batched_tokens=16, max_concurrent=3)
    results = sched.run_all([Request(p, SamplingParams(), max_tokens=7) for p in prompts])
    assert [r.tokens for r in results] == serial
    assert max(len(s) for s in runner.steps) == 3  # never more than max_concurrent live
    assert runner.num_free_blocks() == runner.num_blocks


def test_eos_stops_and_is_not_emitted():
    p = prompt(6, 3)
    free_run = expected_tokens(p, 10)
    eos = free_run[3]
    stop_at = free_run.index(eos)
    runner = FakeRunner()
    result = make(runner, eos_token_id=eos).run(Request(p, SamplingParams(), max_tokens=10))
    assert result.finish_reason == "stop" and result.tokens == free_run[:stop_at]
    ignoring = make(FakeRunner(), eos_token_id=eos).run(
        Request(p, SamplingParams(ignore_eos=True), max_tokens=10))
    assert ignoring.finish_reason == "length" and ignoring.tokens == free_run


def test_empty_prompt_zero_max_tokens_and_cancel():
    sched = make(FakeRunner())
    assert sched.run(Request([], SamplingParams(), max_tokens=5)).finish_reason == "stop"
    assert sched.run(Request([1, 2], SamplingParams(), max_tokens=0)).finish_reason == "length"
    handle = sched.submit(Request(prompt(5, 0), SamplingParams(), max_tokens=100))
    sched.step()
    handle.cancel()
    result = handle.wait()
    assert result.finish_reason == "cancelled" and 1 <= len(result.tokens) < 100
    assert sched.runner.num_free_blocks() == sched.runner.num_blocks


def test_prompt_that_can_never_fit_is_cancelled_others_go_on():
    runner = FakeRunner(num_blocks=4, block_size=4)
    sched = make(runner, decode_headroom_blocks=1)
    big = sched.submit(Request(prompt(17, 0), SamplingParams(), max_tokens=2))
    small = sched.submit(Request(prompt(5, 1), SamplingParams(), max_tokens=2))
    while sched.step():
        pass
    assert big.wait().finish_reason == "cancelled" and big.wait().tokens == []
    assert small.wait().tokens == expected_tokens(prompt(5, 1), 2)
    assert sched.stats["rejected"] == 1


def test_admission_waits_for_pages_and_fills_a_freed_seat():
    runner = FakeRunner(num_blocks=6, block_size=4)
    sched = make(runner, decode_headroom_blocks=1, max_concurrent=4)
    first = sched.submit(Request(prompt(14, 0), SamplingParams(), max_tokens=3))   # 4 pages + 1 headroom
    second = sched.submit(Request(prompt(10, 1), SamplingParams(), max_tokens=3))  # needs 3 + 1: must wait
    sched.step()
    assert [rid for rid, _, _ in runner.steps[0]] == [0]
    while sched.step():
        pass
    assert first.wait().tokens == expected_tokens(prompt(14, 0), 3)
    assert second.wait().tokens == expected_tokens(prompt(10, 1), 3)
    # the second request was admitted in the step right after the first finished
    first_step_of_second = next(i for i, s in enumerate(runner.steps) if any(r == 1 for r, _, _ in s))
    last_step_of_first = max(i for i, s in enumerate(runner.steps) if any(r == 0 for r, _, _ in s))
    assert first_step_of_second == last_step_of_first + 1


def test_out_of_pages_preempts_the_youngest_and_recomputes_it():
    """Decoding outgrows the pool: the youngest request is freed, queued first and
    fed again (prompt + what it generated); every request still gets the tokens it
    would get alone, and nothing is emitted twice."""
    prompts = [prompt(8, 20), prompt(8, 21), prompt(8, 22)]
    runner = FakeRunner(num_blocks=9, block_size=4)
    sched = make(runner, decode_headroom_blocks=0, max_concurrent=3)
    results = sched.run_all([Request(p, SamplingParams(), max_tokens=12) for p in prompts])
    assert sched.stats["preemptions"] >= 1
    for p, result in zip(prompts, results):
        assert result.tokens == expected_tokens(p, 12) and result.finish_reason == "length"
    assert runner.num_free_blocks() == runner.num_blocks
    # a preempted request comes back as a portion longer than its prompt
    assert any(n > 8 for s in runner.steps for _, n, _ in s)


def test_request_that_outgrows_the_whole_pool_alone_is_cancelled_with_what_it_has():
    runner = FakeRunner(num_blocks=3, block_size=4)
    sched = make(runner, decode_headroom_blocks=0)
    result = sched.run(Request(prompt(8, 5), SamplingParams(), max_tokens=50))
    assert result.finish_reason == "cancelled"
    assert result.tokens == expected_tokens(prompt(8, 5), len(result.tokens)) and len(result.tokens) >= 4
    assert runner.num_free_blocks() == runner.num_blocks


def test_sampler_gets_seed_and_draw_index_per_request():
    seen = []

    def sampler(logits, params, seeds, draws):
        seen.append((list(seeds), list(draws), [p.temperature for p in params]))
        return logits.argmax(dim=-1).tolist()

    sched = make(FakeRunner(), sampler=sampler, base_seed=5)
    sched.run_all([
        Request(prompt(4, 0), SamplingParams(temperature=0.8, seed=1234), max_tokens=3),
        Request(prompt(6, 1), SamplingParams(), max_tokens=2),
    ])
    assert seen[0][0][0] == 1234 and seen[0][1] == [0, 0] and seen[0][2] == [0.8, 0.0]
    assert seen[1][1] == [1, 1] and seen[2][1] == [2]
    assert seen[0][0][1] != 1234  # a request without a seed gets one of its own


def test_engine_thread_runs_requests_and_stop_cancels():
    sched = make(FakeRunner())
    sched.start()
    try:
        result = sched.run(Request(prompt(9, 2), SamplingParams(), max_tokens=5))
        assert result.tokens == expected_tokens(prompt(9, 2), 5)
    finally:
        sched.stop()
    assert sched.runner.num_free_blocks() == sched.runner.num_blocks


def test_out_of_memory_with_nothing_to_preempt_is_raised():
    class Broken(FakeRunner):
        def step(self, entries):
            raise OutOfMemoryError("always")

    sched = make(Broken())
    handle = sched.submit(Request(prompt(4, 0), SamplingParams(), max_tokens=2))
    sched.step()  # preempting the only request cancels it
    assert handle.wait().finish_reason == "cancelled"


def test_stream_yields_each_token_then_the_terminal_step():
    # driven by the caller (no engine thread)
    sched = make(FakeRunner())
    steps = list(sched.stream(Request(prompt(7, 5), SamplingParams(), max_tokens=4)))
    assert [s.tokens for s in steps[:-1]] == [(t,) for t in expected_tokens(prompt(7, 5), 4)]
    assert steps[-1].finish_reason == "length" and all(s.finish_reason is None for s in steps[:-1])
    # and with the engine thread, two streams at once
    sched = make(FakeRunner())
    sched.start()
    try:
        first = sched.submit(Request(prompt(5, 6), SamplingParams(), max_tokens=3))
        second = sched.submit(Request(prompt(11, 7), SamplingParams(), max_tokens=6))
        got_second = [s for s in second.stream()]
        got_first = [s for s in first.stream()]
        assert sched.is_running
    finally:
        sched.stop()
    assert not sched.is_running
    assert [t for s in got_first for t in s.tokens] == expected_tokens(prompt(5, 6), 3)
    assert [t for s in got_second for t in s.tokens] == expected_tokens(prompt(11, 7), 6)
    assert got_first[-1].finish_reason == "length" and got_second[-1].finish_reason == "length"


def test_load_stats_counts_queues_and_pages():
    runner = FakeRunner(num_blocks=16, block_size=4, max_concurrent=2)
    sched = make(runner, max_concurrent=2, decode_headroom_blocks=0)
    load = sched.load_stats()
    assert (load.num_waiting, load.num_running, load.kv_cache_usage) == (0, 0, 0.0)
    assert (load.block_size, load.num_blocks) == (4, 16)
    handles = [sched.submit(Request(prompt(8, s), SamplingParams(), max_tokens=50)) for s in range(3)]
    assert sched.load_stats().num_waiting == 3
    sched.step()  # two seats: two admitted and prefilled, one waits
    load = sched.load_stats()
    assert (load.num_waiting, load.num_running) == (1, 2)
    assert load.kv_cache_usage == pytest.approx(4 / 16)  # 2 requests x 8 tokens = 4 pages of 4
    for handle in handles:
        handle.cancel()
    sched.step()
    assert sched.load_stats().kv_cache_usage == 0.0


def test_trace_out_holds_one_event_per_step_with_its_kind_and_sizes(tmp_path):
    # one duration event per step that ran the model, as the reference records them
    # (scheduler/continuous_scheduler.py:502-527): B, phase, total_q
    path = tmp_path / "steps.json"
    runner = FakeRunner()
    sched = make(runner, chunk_size=4, max_num_batched_tokens=6, trace_out=str(path))
    handles = [sched.submit(Request(prompt(n, n), SamplingParams(), max_tokens=3)) for n in (3, 7)]
    while sched.step():
        pass
    for handle in handles:
        handle.wait()
    sched.stop()  # no thread was started: only writes the trace
    import json

    events = json.loads(path.read_text())["traceEvents"]
    assert len(events) == len(runner.steps) == sched.stats["steps"]
    assert [e["args"]["B"] for e in events] == [len(s) for s in runner.steps]
    assert [e["args"]["total_q"] for e in events] == [sum(n for _, n, _ in s) for s in runner.steps]
    # step 0: both prompts' first portions (3 whole + 3 of 7); step 1: a decoded token beside a portion
    assert events[0]["args"]["phase"] == "prefill"
    assert events[1]["args"]["phase"] == "mixed"
    assert events[-1]["args"]["phase"] == "decode"
    assert all(e["ph"] == "X" and e["name"] == "step" and e["dur"] >= 0 for e in events)
    assert events[0]["ts"] == 0 and all(a["ts"] <= b["ts"] for a, b in zip(events, events[1:]))


# -- a step that fails leaves the cache as it was ------------------------------------------------


class _FailingModel:
    """Stands where a `DecoderModel` stands in a `ModelRunner`: logits of zeros, or an error on demand."""

    graph_safe = False
    dtype = torch.float32
    device = torch.device("cpu")

    vocab_size = VOCAB

    def __init__(self, needs=None):
        self.fail_with = None
        self.positions_seen = []
        self.needs = needs if needs is not None else [CacheNeeds(pages=PagedKVNeeds(1, 16))]

    def cache_needs(self, page_size):
        return self.needs

    def forward(self, ctx, caches):
        # a mixer with state of fixed size updates it in place as it goes: every request's row
        # of every state tensor counts the tokens the request has brought so far
        for cache in caches:
            tensors = cache.state.values() if isinstance(cache.state, dict) else [cache.state] if cache.state is not None else []
            for tensor in tensors:
                for b, slot in enumerate(ctx.host_state_slots):
                    tensor[slot] += ctx.host_cu_seqlens_q[b + 1] - ctx.host_cu_seqlens_q[b]
        if self.fail_with is not None:
            raise self.fail_with
        self.positions_seen.append(ctx.positions.tolist())
        return torch.zeros((ctx.logit_rows.numel(), VOCAB))


def test_a_step_that_raises_leaves_lengths_pages_and_admissions_as_they_were():
    from mini_infer_amd.engine.batch import StepEntry
    from mini_infer_amd.engine.model_runner import ModelRunner
    from mini_infer_amd.exceptions import KernelShapeError

    model = _FailingModel()
    runner = ModelRunner(model, None, num_blocks=8, block_size=4, max_concurrent=3, cuda_graph=False)
    runner.step([StepEntry("old", [1, 2, 3, 4, 5, 6], [5])])
    free_before = runner.num_free_blocks()
    assert free_before == 8 - 2 and runner.cache.length("old") == 6

    model.fail_with = KernelShapeError("a kernel refuses this size")
    with pytest.raises(KernelShapeError):
        # "old" would grow into a third page, "new" would be admitted with two pages
        runner.step([StepEntry("old", [7, 8, 9], [2]), StepEntry("new", [1, 2, 3, 4, 5], [4])])
    runner.cache.check()
    assert runner.num_free_blocks() == free_before
    assert runner.cache.length("old") == 6 and not runner.has_request("new")
    assert runner.cache.states.num_free == 2

    model.fail_with = None
    runner.step([StepEntry("old", [7, 8, 9], [2]), StepEntry("new", [1, 2, 3], [2])])
    assert model.positions_seen[-1] == [6, 7, 8, 0, 1, 2]
    assert runner.cache.length("old") == 9 and runner.cache.length("new") == 3
    runner.cache.check()
    runner.free_request("old")
    runner.free_request("new")
    assert runner.num_free_blocks() == 8


def test_a_step_that_raises_leaves_state_of_fixed_size_bit_equal():
    """A model with pages and with two state tensors of different shapes and dtypes per call:
    the failing step has already added to the state rows of its requests (and would have
    written their positions) when it raises; afterwards every state tensor and the slot table
    hold what they held before, and a request the step had admitted is gone."""
    from mini_infer_amd.engine.batch import StepEntry
    from mini_infer_amd.engine.model_runner import ModelRunner
    from mini_infer_amd.exceptions import KernelShapeError
    from mini_infer_amd.parts.base import StateNeeds

    needs = [
        CacheNeeds(pages=PagedKVNeeds(1, 16), state=StateNeeds((3,))),
        CacheNeeds(state={"tail": StateNeeds((2, 2), torch.bfloat16), "recurrent": StateNeeds((5,), torch.float64)}),
    ]
    model = _FailingModel(needs)
    runner = ModelRunner(model, None, num_blocks=8, block_size=4, max_concurrent=3, cuda_graph=False)
    caches = runner._layer_caches
    assert caches[0].state.shape == (4, 3) and caches[0].state.dtype == torch.float32
    assert set(caches[1].state) == {"tail", "recurrent"}
    assert caches[1].state["tail"].shape == (4, 2, 2) and caches[1].state["tail"].dtype == torch.bfloat16
    assert caches[1].state["recurrent"].shape == (4, 5) and caches[1].state["recurrent"].dtype == torch.float64
    runner.step([StepEntry("old", [1, 2, 3, 4, 5, 6], [5]), StepEntry("other", [9, 9], [])])
    slot = runner.cache.state_slot("old")
    assert caches[0].state[slot].tolist() == [6.0] * 3 and caches[1].state["recurrent"][slot].tolist() == [6.0] * 5

    def everything():
        # (the host's copy of the slot table: without a GPU no kernel writes the device's)
        tensors = [caches[0].state, caches[1].state["tail"], caches[1].state["recurrent"]]
        return [t.clone() for t in tensors] + [torch.from_numpy(runner.cache.states.host[[slot]].copy())]

    before = everything()
    model.fail_with = KernelShapeError("a kernel refuses this size")
    with pytest.raises(KernelShapeError):
        runner.step([StepEntry("old", [7, 8, 9], [2]), StepEntry("new", [1, 2, 3, 4, 5], [4])])
    for was, now in zip(before, everything()):
        assert torch.equal(was, now)
    runner.cache.check()
    assert runner.cache.length("old") == 6 and not runner.has_request("new") and runner.cache.states.num_free == 1
    model.fail_with = None
    runner.step([StepEntry("old", [7, 8, 9], [2])])
    assert caches[0].state[slot].tolist() == [9.0] * 3 and caches[1].state["tail"][slot].float().flatten().tolist() == [9.0] * 4


def test_a_failing_device_copy_during_rollback_still_frees_everything_and_reports_the_first_error(monkeypatch):
    """The rollback of a failed step puts the host's books right before it touches the device;
    if sending the positions back fails too (the device is what broke), pages and admissions
    are back all the same and the step's own error is the one raised."""
    from mini_infer_amd.engine.batch import StepEntry
    from mini_infer_amd.engine.model_runner import ModelRunner
    from mini_infer_amd.exceptions import KernelShapeError

    model = _FailingModel()
    runner = ModelRunner(model, None, num_blocks=8, block_size=4, max_concurrent=3, cuda_graph=False)
    runner.step([StepEntry("old", [1, 2, 3, 4, 5, 6], [5])])
    model.fail_with = KernelShapeError("the step's own error")

    def broken(slot):
        raise RuntimeError("the device is gone")

    monkeypatch.setattr(runner.cache.states, "push_position", broken)
    with pytest.raises(KernelShapeError, match="the step's own error"):
        runner.step([StepEntry("old", [7, 8, 9], [2]), StepEntry("new", [1, 2, 3, 4, 5], [4])])
    runner.cache.check()
    assert runner.num_free_blocks() == 6 and not runner.has_request("new") and runner.cache.states.num_free == 2


class StateOnlyRunner(FakeRunner):
    """A runner whose model keeps no pages at all: state of fixed size per request only."""

    def __init__(self, max_concurrent=2):
        from mini_infer_amd.parts.base import StateNeeds

        self.num_blocks, self.block_size = 16, 4
        self.cache = CacheManager([CacheNeeds(state=StateNeeds((4,)))], page_size=4, num_pages=16,
                                  max_requests=max_concurrent, allocate_storage=False)
        self.history, self.steps = {}, []

    def num_free_blocks(self):
        return self.num_blocks  # what `ModelRunner.num_free_blocks` answers without page groups


def test_a_model_whose_only_cache_is_state_of_fixed_size_is_admitted_by_seats_and_finishes():
    """No page group: admission goes by seats alone, prompts of any length are taken, the
    requests run and finish, the third waits for a seat (it does not wait for pages for ever)."""
    runner = StateOnlyRunner(max_concurrent=2)
    assert not runner.cache.has_pages and runner.cache.pages_for_tokens(1000) == 0
    sched = make(runner, max_concurrent=2, chunk_size=16, max_num_batched_tokens=32)
    lengths = (70, 3, 200)  # far more tokens than 16 pages of 4 would hold
    handles = [sched.submit(Request(prompt(n, n), SamplingParams(), max_tokens=5)) for n in lengths]
    for _ in range(200):
        if not sched.step() and not sched.has_work():
            break
    assert all(h.done() for h in handles)
    for handle, n in zip(handles, lengths):
        result = handle.wait()
        assert result.finish_reason == "length" and result.tokens == expected_tokens(prompt(n, n), 5)
    assert max(len(step) for step in runner.steps) == 2  # never more requests than seats
    assert sched.stats["preemptions"] == 0 and sched.stats["rejected"] == 0
    assert runner.cache.states.num_free == 2
    assert sched.load_stats().kv_cache_usage == 0.0


def test_a_request_past_the_models_positions_is_cancelled_and_counted():
    """`max_position_embeddings` bounds admission: a request whose prompt and `max_tokens`
    together would feed a position past it ends as cancelled, with a reason of its own in the
    statistics; one that just fits runs."""
    runner = FakeRunner()
    runner.max_model_len = 20
    sched = make(runner)
    fits = sched.submit(Request(prompt(12, 1), SamplingParams(), max_tokens=9))  # feeds positions 0..19
    too_long = sched.submit(Request(prompt(12, 2), SamplingParams(), max_tokens=10))
    long_prompt = sched.submit(Request(prompt(30, 3), SamplingParams(), max_tokens=1))
    while sched.step():
        pass
    assert fits.wait().finish_reason == "length" and len(fits.wait().tokens) == 9
    assert too_long.wait().finish_reason == "cancelled" and too_long.wait().tokens == []
    assert long_prompt.wait().finish_reason == "cancelled"
    assert sched.stats["rejected_too_long"] == 2 and sched.stats["rejected"] == 0
    assert runner.num_free_blocks() == runner.num_blocks


def test_an_oversubscribed_load_is_admitted_in_waves_without_preemption():
    """Sixteen long prompts for a pool that holds eight: admission counts the pages that the
    requests already admitted will still take, so the rest waits instead of being admitted,
    preempted and recomputed."""
    runner = FakeRunner(num_blocks=4096, block_size=4, max_concurrent=16)
    sched = make(runner, max_concurrent=16, chunk_size=512, max_num_batched_tokens=2048)
    prompts = [prompt(2000, 100 + i) for i in range(16)]
    handles = [sched.submit(Request(p, SamplingParams(), max_tokens=12)) for p in prompts]
    most_live = 0
    while sched.step():
        most_live = max(most_live, len(runner.cache.live_requests()))
    assert sched.stats["preemptions"] == 0 and sched.stats["rejected"] == 0
    assert most_live == 8  # 500 pages of prompt + 3 of decoding each (8 of headroom asked for)
    assert sched.stats["tokens_run"] == sum(len(p) + 11 for p in prompts)  # nothing was fed twice
    for handle, p in zip(handles, prompts):
        assert handle.wait().tokens == expected_tokens(p, 12)
    assert runner.num_free_blocks() == runner.num_blocks


def test_draw_index_lives_in_the_state_slot_survives_preemption_and_starts_at_zero_in_a_reused_slot():
    """What the sampler is told comes from the request's state slot.  A preempted request is
    given another slot when it returns and goes on with the draw index it had reached; a slot
    that a finished request leaves starts at draw 0 for the next one."""
    draws_by_seed: dict[int, list[int]] = {}
    slot_rows = []

    def sampler(logits, params, seeds, draws):
        for seed, draw in zip(seeds, draws):
            draws_by_seed.setdefault(seed, []).append(draw)
        return logits.argmax(dim=-1).tolist()

    prompts = [prompt(8, 20), prompt(8, 21), prompt(8, 22)]
    runner = FakeRunner(num_blocks=9, block_size=4, max_concurrent=3)
    sched = make(runner, sampler=sampler, decode_headroom_blocks=0, max_concurrent=3)
    requests = [Request(p, SamplingParams(temperature=0.5, top_k=7, top_p=0.9, seed=1000 + i), max_tokens=12)
                for i, p in enumerate(prompts)]
    handles = [sched.submit(r) for r in requests]
    sched.step()
    states = runner.cache.states
    for i in range(3):  # settings and seed are in the slot's row, the position follows the cache
        slot = runner.cache.state_slot(i)
        slot_rows.append(states.host[slot].copy())
        assert states.seed(slot) == 1000 + i and states.position(slot) == runner.cache.length(i) == 8
        assert states.host[slot, 5] == 7 and states.draws(slot) == 1
        assert np.array([0.5, 0.9], dtype=np.float32).view(np.int32).tolist() == [states.host[slot, 4], states.host[slot, 6]]
    while sched.step():
        pass
    assert sched.stats["preemptions"] >= 1
    for i, (p, handle) in enumerate(zip(prompts, handles)):
        assert handle.wait().tokens == expected_tokens(p, 12)
        assert draws_by_seed[1000 + i] == list(range(12))  # no draw index used twice or skipped
    # every slot is free again; the next request finds draw 0 and its own settings, not the last owner's
    assert states.num_free == 3
    sched.submit(Request(prompt(5, 1), SamplingParams(seed=77), max_tokens=1))
    sched._admit_waiting()
    slot = runner.cache.state_slot(3)
    assert states.draws(slot) == 0 and states.seed(slot) == 77 and states.position(slot) == 0
    assert states.host[slot, 5] == 0 and states.host[slot, 4] == 0


@pytest.mark.parametrize("seed", range(120))
def test_random_loads_give_every_request_the_tokens_it_would_get_alone(seed):
    """Random loads on random small engines (pools from barely enough to plenty, budgets, portion
    sizes, seats, headroom, an end-of-sequence token or none): whatever the scheduler decides
    (portions, waves of admission, preemption and recomputation, cancelling what can never
    fit), a request that ends by itself has exactly the tokens it would get alone, one that is
    cancelled has a prefix of them, no step breaks the budget or the seats, and every page
    and slot comes back."""
    rng = np.random.default_rng(1000 + seed)
    block_size = int(rng.choice([2, 4, 8]))
    num_blocks = int(rng.integers(6, 60))
    max_concurrent = int(rng.integers(1, 7))
    budget = int(rng.integers(4, 40))
    chunk = int(rng.integers(2, 40))
    eos = int(rng.integers(0, VOCAB)) if rng.random() < 0.5 else None
    runner = FakeRunner(num_blocks=num_blocks, block_size=block_size, max_concurrent=max_concurrent)
    sched = make(runner, chunk_size=chunk, max_num_batched_tokens=budget, max_concurrent=max_concurrent,
                 decode_headroom_blocks=int(rng.integers(0, 3)), eos_token_id=eos)
    requests = [Request(prompt(int(rng.integers(1, 50)), seed * 100 + i),
                        SamplingParams(ignore_eos=bool(rng.random() < 0.2)), max_tokens=int(rng.integers(0, 24)))
                for i in range(int(rng.integers(1, 13)))]
    results = sched.run_all(requests)
    assert len(results) == len(requests)
    for request, result in zip(requests, results):
        alone = expected_tokens(request.prompt, request.max_tokens, None if request.sampling_params.ignore_eos else eos)
        if result.finish_reason == "cancelled":
            assert result.tokens == alone[: len(result.tokens)]
        else:
            assert result.tokens == alone
            assert result.finish_reason == ("length" if len(alone) == request.max_tokens else "stop")
    for step in runner.steps:
        assert len(step) <= max_concurrent and sum(n for _, n, _ in step) <= budget
        assert len({rid for rid, _, _ in step}) == len(step)  # a request is in a step once
    runner.cache.check()
    assert runner.num_free_blocks() == num_blocks and runner.cache.states.num_free == max_concurrent
