"""Continuous batching above the step function.

Each step: finished requests have already given their pages back; waiting
requests are admitted first-come-first-served while a seat and enough pages are
free; then ONE batch is built under a token budget: every decoding request feeds
its last token, and what is left of the budget is handed to prefilling requests
in admission order as portions of their prompts, cut wherever the budget ends.
The step runs, and every request whose last fed token completed what it had to
feed gets its next token sampled on the device.

Names and policies follow the reference's `ContinuousScheduler`
(scheduler/continuous_scheduler.py): `max_concurrent`, `decode_headroom_blocks`,
`chunk_size` (:144-177); FIFO admission by block budget, with a prompt that can
never fit finished as "cancelled" (:670-773); EOS ends with "stop" and is not
emitted, `max_tokens` ends with "length", the last emitted token is never fed
(:847-860).  Two things differ by design:
  * a global token budget per step (`max_num_batched_tokens`); the reference only
    bounds each request's chunk;
  * when pages run out mid-flight, the youngest running request is preempted and
    recomputed later (its pages are freed, it goes back to the FRONT of the
    queue and feeds prompt + generated tokens again), so no request is lost and
    greedy and seeded outputs are unchanged.  The reference cancels the youngest
    request instead (:388-416).  A request that cannot fit even alone is
    finished as "cancelled".

Asynchronous sampling (the reference's `async_sampling`, :529-646): tokens are sampled on
the device and the NEXT step is launched from them while they are still there; the host
reads a step's ids one step late, so its work (bookkeeping, building the next batch)
overlaps the device's.  End-of-sequence is therefore seen one step late: the request has
been fed once more by then, and that step's result for it is dropped.  Outputs are the
same as without it.
"""

from __future__ import annotations

import collections
import dataclasses
import json
import threading
import time
from typing import Any, Callable, Iterable, Iterator, Sequence

from mini_infer_amd.config.engine_config import DEFAULT_CHUNK_SIZE, DEFAULT_DECODE_HEADROOM_BLOCKS, EngineConfig
from mini_infer_amd.engine.batch import StepEntry
from mini_infer_amd.engine.request import (
    GenerationResult,
    GenerationStep,
    Request,
    RequestState,
    RunningRequest,
)
from mini_infer_amd.exceptions import EngineNotRunningError, OutOfMemoryError

IDLE_SLEEP_SECONDS = 0.005


@dataclasses.dataclass(frozen=True)
class SchedulerLoad:
    """Queue lengths and cache use at one moment (the reference's `load_stats`,
    scheduler/continuous_scheduler.py:280-300)."""

    num_waiting: int
    num_running: int
    kv_cache_usage: float
    block_size: int
    num_blocks: int


@dataclasses.dataclass
class _PendingSample:
    """Ids sampled by the last step that the host has not read yet."""

    requests: list[RunningRequest]  # row i belongs to requests[i]
    on_device: Any  # int32 tensor [rows]
    on_host: Any  # pinned int32 tensor [rows], valid once `copied` has happened
    copied: Any  # event


class RequestHandle:
    """What `submit` returns: wait for the result or walk the steps so far."""

    def __init__(self, scheduler: "ContinuousScheduler", running: RunningRequest) -> None:
        self._scheduler = scheduler
        self._running = running

    @property
    def request_id(self) -> int:
        return self._running.request_id

    def done(self) -> bool:
        return self._running.done_event.is_set()

    def cancel(self) -> None:
        self._running.cancel_requested = True

    def wait(self, timeout: float | None = None) -> GenerationResult:
        deadline = None if timeout is None else time.time() + timeout
        while not self._running.done_event.wait(0.05):
            if self._scheduler._thread is not None and not self._scheduler.engine_alive:
                raise EngineNotRunningError("the engine stopped before the request finished")
            if self._scheduler._thread is None:
                # no engine thread: drive the engine from the caller
                self._scheduler.step()
            if deadline is not None and time.time() > deadline:
                raise TimeoutError("request did not finish in time")
        return self._scheduler._result_of(self._running)

    def steps(self) -> list[GenerationStep]:
        return list(self._running.steps)

    def stream(self, poll_seconds: float = 0.002) -> Iterator[GenerationStep]:
        """The request's steps as the engine produces them, the terminal one (with its
        `finish_reason`) last; as the reference's `RequestHandle.steps()`
        (scheduler/continuous_scheduler.py:195-204).  Without an engine thread the caller
        drives the engine while it waits."""
        sent = 0
        while True:
            produced = self._running.steps
            while sent < len(produced):
                step = produced[sent]
                sent += 1
                yield step
                if step.finish_reason is not None:
                    return
            if self._scheduler._thread is None:
                if not self._scheduler.step() and not self._scheduler.has_work() and sent >= len(self._running.steps):
                    raise EngineNotRunningError("the request was never finished and the engine has no work left")
            else:
                if not self._scheduler.engine_alive and sent >= len(self._running.steps):
                    raise EngineNotRunningError("the engine stopped before the request finished")
                time.sleep(poll_seconds)


class ContinuousScheduler:
    def __init__(
        self,
        runner: Any,
        max_concurrent: int = 16,
        decode_headroom_blocks: int = DEFAULT_DECODE_HEADROOM_BLOCKS,
        chunk_size: int = DEFAULT_CHUNK_SIZE,
        max_num_batched_tokens: int = 2048,
        *,
        eos_token_id: int | Sequence[int] | None = None,
        tokenizer: Any = None,
        base_seed: int = 0,
        sampler: Callable[..., list[int]] | None = None,
        async_sampling: bool | None = None,
        trace_out: str | None = None,
    ) -> None:
        if max_concurrent <= 0 or chunk_size <= 0 or max_num_batched_tokens <= 0:
            raise ValueError("max_concurrent, chunk_size and max_num_batched_tokens must be positive")
        if decode_headroom_blocks < 0:
            raise ValueError("decode_headroom_blocks must be >= 0")
        self.runner = runner
        self.cache = runner.cache
        self.max_concurrent = max_concurrent
        self.decode_headroom_blocks = decode_headroom_blocks
        self.chunk_size = chunk_size
        self.max_num_batched_tokens = max_num_batched_tokens
        if eos_token_id is None:
            self.eos_token_ids: frozenset[int] = frozenset()
        elif isinstance(eos_token_id, int):
            self.eos_token_ids = frozenset([eos_token_id])
        else:
            self.eos_token_ids = frozenset(int(t) for t in eos_token_id)
        self.tokenizer = tokenizer
        self.base_seed = base_seed
        # None: the device's own sampler, which reads every request's settings, seed and draw
        # index from its state slot; a callable `(logits, params, seeds, draws) -> ids` replaces it
        self._sample = sampler
        # None: on where it can be (the runner takes tokens from the device and the sampler is the device's own)
        can_async = sampler is None and bool(getattr(runner, "supports_device_tokens", False))
        if async_sampling and not can_async:
            raise ValueError("async_sampling needs a runner that takes device tokens and the built-in sampler")
        self.async_sampling = can_async if async_sampling is None else bool(async_sampling)
        self._pending: _PendingSample | None = None
        self._ids_on_host = None  # pinned int32 [max_concurrent], made at the first asynchronous sample
        self._ids_copied = None  # event after the copy into it
        self._waiting: collections.deque[RunningRequest] = collections.deque()
        self._running: list[RunningRequest] = []
        self._next_id = 0
        self._admitted = 0
        self._lock = threading.Lock()
        self._thread: threading.Thread | None = None
        self._stop = threading.Event()
        self._crashed: BaseException | None = None
        # `rejected`: requests that could never fit the page pool; `rejected_too_long`: requests
        # whose prompt and `max_tokens` together pass the positions the model was made for
        self.stats = {"steps": 0, "preemptions": 0, "tokens_run": 0, "rejected": 0, "rejected_too_long": 0}
        # the most positions a request may reach (the model's `max_position_embeddings`), or None
        self.max_model_len: int | None = getattr(runner, "max_model_len", None)
        # A timeline of the steps in the Chrome trace-event format, as the reference records
        # it (scheduler/continuous_scheduler.py:223-229, :502-527): one duration event per
        # step that ran the model, written by `stop()` or `write_trace()`.
        self.trace_out = trace_out
        self._trace_events: list[dict[str, Any]] | None = [] if trace_out is not None else None
        self._trace_start: float | None = None

    @classmethod
    def from_config(cls, runner: Any, engine: EngineConfig, **others: Any) -> "ContinuousScheduler":
        """A scheduler with the knobs of `engine`; `others` are what an `EngineConfig` does not
        hold (`eos_token_id`, `tokenizer`, `sampler`)."""
        return cls(
            runner,
            max_concurrent=engine.max_concurrent,
            decode_headroom_blocks=engine.decode_headroom_blocks,
            chunk_size=engine.chunk_size,
            max_num_batched_tokens=engine.max_num_batched_tokens,
            base_seed=engine.seed,
            async_sampling=engine.async_sampling,
            trace_out=engine.trace_out,
            **others,
        )

    # -- submitting -----------------------------------------------------------

    def _tokenize(self, prompt: str | Sequence[int]) -> list[int]:
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise ValueError("a text prompt needs a tokenizer; pass token ids instead")
            return list(self.tokenizer.encode(prompt))
        return [int(t) for t in prompt]

    def submit(self, request: Request) -> RequestHandle:
        if self._crashed is not None:
            raise EngineNotRunningError(f"the engine has failed: {self._crashed!r}")
        with self._lock:
            request_id = self._next_id
            self._next_id += 1
        seed = request.sampling_params.seed
        if seed is None:
            seed = (self.base_seed * 0x9E3779B97F4A7C15 + request_id) & 0xFFFFFFFFFFFFFFFF
        running = RunningRequest(
            request_id=request_id,
            request=request,
            prompt_token_ids=self._tokenize(request.prompt),
            seed=seed,
        )
        with self._lock:
            self._waiting.append(running)
        return RequestHandle(self, running)

    def run(self, request: Request) -> GenerationResult:
        return self.submit(request).wait()

    def stream(self, request: Request) -> Iterator[GenerationStep]:
        """Submit and yield each generation step as the engine produces it."""
        yield from self.submit(request).stream()

    def load_stats(self) -> SchedulerLoad:
        """Queue lengths and cache use now; callable from any thread (a value may be one step old)."""
        running = sum(1 for r in list(self._running) if r.state != RequestState.DONE)
        num_blocks = self.runner.num_blocks
        return SchedulerLoad(
            num_waiting=len(self._waiting),
            num_running=running,
            kv_cache_usage=1.0 - self._free_pages() / num_blocks if num_blocks else 0.0,
            block_size=self.runner.block_size,
            num_blocks=num_blocks,
        )

    @property
    def is_running(self) -> bool:
        """Whether the engine thread is alive (False before `start`, after `stop`, after a crash)."""
        return self.engine_alive

    def run_all(self, requests: Iterable[Request]) -> list[GenerationResult]:
        """Submit all, drive the engine until all are done; results in submission order."""
        handles = [self.submit(r) for r in requests]
        if self._thread is None:
            while not all(h.done() for h in handles):
                if not self.step() and not self.has_work():
                    break
        return [h.wait() for h in handles]

    # -- engine thread (optional) -------------------------------------------------

    @property
    def engine_alive(self) -> bool:
        return self._thread is not None and self._thread.is_alive() and self._crashed is None

    def start(self) -> None:
        if self._thread is not None:
            return
        self._stop.clear()
        self._thread = threading.Thread(target=self._engine_loop, name="mini-infer-engine", daemon=True)
        self._thread.start()

    def stop(self) -> None:
        thread = self._thread
        if thread is None:
            self.write_trace()
            return
        self._stop.set()
        thread.join()
        self._thread = None
        for running in list(self._running) + list(self._waiting):
            self._finish(running, "cancelled")
        self._running.clear()
        self._waiting.clear()
        self._pending = None
        self.write_trace()

    def trace_events(self) -> list[dict[str, Any]]:
        """The step events recorded so far (empty without `trace_out`)."""
        return list(self._trace_events or [])

    def write_trace(self) -> None:
        """Write the steps recorded so far to `trace_out` (nothing without it)."""
        if self._trace_events is not None and self.trace_out is not None:
            with open(self.trace_out, "w") as f:
                json.dump({"traceEvents": self._trace_events}, f)

    def _record_step(self, started: float, entries: list[StepEntry]) -> None:
        """One "X" event: host time from building the batch to the end of the step's
        bookkeeping, with the number of requests, the tokens run and the kind of step
        (`prefill`: portions of prompts only, `decode`: single tokens only, else `mixed`)."""
        if self._trace_events is None:
            return
        if self._trace_start is None:
            self._trace_start = started
        single = sum(1 for e in entries if len(e.tokens) == 1 and e.want)
        phase = "decode" if single == len(entries) else ("prefill" if single == 0 else "mixed")
        self._trace_events.append(
            {
                "name": "step",
                "ph": "X",
                "ts": (started - self._trace_start) * 1e6,
                "dur": (time.perf_counter() - started) * 1e6,
                "pid": 0,
                "tid": 0,
                "args": {"B": len(entries), "phase": phase, "total_q": sum(len(e.tokens) for e in entries)},
            }
        )

    def _engine_loop(self) -> None:
        try:
            while not self._stop.is_set():
                if not self.step():
                    time.sleep(IDLE_SLEEP_SECONDS)
        except BaseException as err:  # noqa: BLE001
            self._crashed = err
            for running in list(self._running) + list(self._waiting):
                self._finish(running, "cancelled")
            raise

    # -- one step -------------------------------------------------------------------

    def has_work(self) -> bool:
        return bool(self._waiting or self._running or self._pending is not None)

    def step(self) -> bool:
        """Admit, build one batch, run it, sample, finish.  False when there was nothing to do."""
        started = time.perf_counter()
        self._cancel_pending()
        self._admit_waiting()
        if not self._running:
            return self._resolve_pending()
        while True:
            entries, owners = self._build_batch()
            if not entries:
                return self._resolve_pending()
            try:
                device_tokens = self._pending.on_device if any(e.device_row is not None for e in entries) else None
                if device_tokens is not None:
                    logits = self.runner.step(entries, device_tokens=device_tokens)
                else:
                    logits = self.runner.step(entries)
                break
            except OutOfMemoryError:
                # what is still on the device is read first, so that a preempted request
                # keeps every token it has been given
                self._resolve_pending()
                if not self._preempt_youngest():
                    raise
        self.stats["steps"] += 1
        self.stats["tokens_run"] += sum(len(e.tokens) for e in entries)
        sampled_for: list[RunningRequest] = []
        for entry, running in zip(entries, owners):
            running.tokens_fed += len(entry.tokens)
            if entry.want:
                sampled_for.append(running)
        # the ids of the step before this one have had this step's launch to arrive
        self._resolve_pending()
        for running in owners:
            if running.state != RequestState.DONE:
                running.state = (
                    RequestState.DECODING if running.prefill_remaining == 0 else RequestState.CHUNKED_PREFILLING
                )
        if sampled_for:
            # (rows of requests that the late ids have just finished are sampled too and dropped)
            if self.async_sampling:
                self._sample_later(logits, sampled_for)
            else:
                token_ids = self._sample_now(logits, sampled_for)
                for running, token in zip(sampled_for, token_ids):
                    if running.state != RequestState.DONE:
                        self._accept_token(running, int(token))
        self._reap_done()
        self._record_step(started, entries)
        return True

    # -- asynchronous sampling ---------------------------------------------------------------

    def _count_draws(self, sampled_for) -> None:
        """The host's copy of each sampled request's draw index follows the device's."""
        for running in sampled_for:
            if running.state != RequestState.DONE and self.cache.has_request(running.request_id):
                self.cache.states.count_draw(self.cache.state_slot(running.request_id))

    def _sample_on_device(self, logits, sampled_for):
        """One id per row, as an int32 device tensor: settings, seed and draw index of every
        row come from its request's state slot, whose draw index the kernel advances."""
        from mini_infer_amd.sampling.sampler import sample_from_slots

        on_device = sample_from_slots(logits, self.runner.last_row_slots, self.cache.states.table)
        self._count_draws(sampled_for)
        return on_device

    def _sample_now(self, logits, sampled_for) -> list[int]:
        if self._sample is None:
            return self._sample_on_device(logits, sampled_for).tolist()
        states = self.cache.states
        slots = [
            self.cache.state_slot(r.request_id) if self.cache.has_request(r.request_id) else None for r in sampled_for
        ]
        params = [r.request.sampling_params for r in sampled_for]
        seeds = [r.seed for r in sampled_for]
        draws = [states.draws(slot) if slot is not None else 0 for slot in slots]
        token_ids = self._sample(logits, params, seeds, draws)
        self._count_draws(sampled_for)
        return token_ids

    def _sample_later(self, logits, sampled_for) -> None:
        """Sample on the device, start the copy of the ids to the host, read nothing yet."""
        import torch

        on_device = self._sample_on_device(logits, sampled_for)
        # One pinned buffer and one event for the scheduler's life: the ids of a step are read
        # (`_resolve_pending`) before the next step's ids are copied into the same place.
        if self._ids_on_host is None or self._ids_on_host.numel() < on_device.numel():
            self._ids_on_host = torch.empty(max(self.max_concurrent, on_device.numel()), dtype=torch.int32, pin_memory=True)
            self._ids_copied = torch.cuda.Event()
        on_host = self._ids_on_host[: on_device.numel()]
        on_host.copy_(on_device, non_blocking=True)
        copied = self._ids_copied
        copied.record()
        for row, running in enumerate(sampled_for):
            if running.state != RequestState.DONE:
                running.pending_row = row
        self._pending = _PendingSample(list(sampled_for), on_device, on_host, copied)

    def _resolve_pending(self) -> bool:
        """Read the ids still on their way and give each request its token.  False if there were none."""
        pending, self._pending = self._pending, None
        if pending is None:
            return False
        pending.copied.synchronize()
        for running, token in zip(pending.requests, pending.on_host.tolist()):
            if running.pending_row is None:
                continue  # finished or cancelled since
            running.pending_row = None
            if running.state != RequestState.DONE:
                self._accept_token(running, int(token))
        self._reap_done()
        return True

    # -- pieces of a step ---------------------------------------------------------------

    def _cancel_pending(self) -> None:
        for running in list(self._running):
            if running.cancel_requested:
                self._finish(running, "cancelled")
        with self._lock:
            waiting = list(self._waiting)
        for running in waiting:
            if running.cancel_requested:
                with self._lock:
                    self._waiting.remove(running)
                self._finish(running, "cancelled")
        self._reap_done()

    def _pages_for(self, tokens: int) -> int:
        return self.cache.pages_for_tokens(tokens)

    def _free_pages(self) -> int:
        return self.runner.num_free_blocks()

    def _promised_pages(self) -> int:
        """Pages that requests already admitted will still take for the tokens they have not
        fed yet (admission reserves nothing, so the pool's free count does not show them)."""
        promised = 0
        for running in self._running:
            remaining = running.prefill_remaining
            if remaining > 0 and self.cache.has_request(running.request_id):
                promised += max(self.cache.pages_needed(running.request_id, remaining), default=0)
        return promised

    def _admit_waiting(self) -> None:
        while len(self._running) < self.max_concurrent:
            with self._lock:
                if not self._waiting:
                    return
                running = self._waiting[0]
            if running.cancel_requested:
                with self._lock:
                    self._waiting.popleft()
                self._finish(running, "cancelled")
                continue
            if not running.prompt_token_ids:
                with self._lock:
                    self._waiting.popleft()
                self._finish(running, "stop")
                continue
            if running.request.max_tokens <= 0:
                with self._lock:
                    self._waiting.popleft()
                self._finish(running, "length")
                continue
            to_feed = len(running.feed)
            remaining_new = running.request.max_tokens - len(running.tokens_generated)
            # positions the request would reach: everything it feeds (the last token it is
            # given is never fed) must lie inside what the model's position encoding was made for
            if self.max_model_len is not None and to_feed + remaining_new - 1 > self.max_model_len:
                with self._lock:
                    self._waiting.popleft()
                self.stats["rejected_too_long"] += 1
                self._finish(running, "cancelled")
                continue
            need_now = self._pages_for(to_feed)
            if need_now > self.runner.num_blocks:
                # can never fit, not even alone
                with self._lock:
                    self._waiting.popleft()
                self.stats["rejected"] += 1
                self._finish(running, "cancelled")
                continue
            # the prompt plus some runway for decoding, but never more than it can ever use
            required = max(
                need_now,
                min(need_now + self.decode_headroom_blocks, self._pages_for(to_feed + remaining_new - 1)),
            )
            # what is free, less what the requests admitted before this one are about to take
            free = self._free_pages() - self._promised_pages()
            if free < required and (self._running or free < need_now):
                return
            with self._lock:
                self._waiting.popleft()
            self.cache.add_request(running.request_id)
            # the request's sampling state lives in its slot; a request that comes back after a
            # preemption goes on with the draw index it had reached
            params = running.request.sampling_params
            self.cache.set_sampling(
                running.request_id, temperature=params.temperature, top_k=params.top_k, top_p=params.top_p,
                seed=running.seed, draw=running.draws,
            )
            running.state = RequestState.PREFILLING
            running.tokens_fed = 0
            running.admitted_order = self._admitted
            self._admitted += 1
            self._running.append(running)

    def _build_batch(self) -> tuple[list[StepEntry], list[RunningRequest]]:
        budget = self.max_num_batched_tokens
        entries: list[StepEntry] = []
        owners: list[RunningRequest] = []
        # a request whose newest token is still on the device decodes from there, unless that
        # token is its last (then it ends when the token is read and is fed nothing more)
        on_device = [r for r in self._running if r.pending_row is not None]
        decoders = [r for r in self._running if r.pending_row is None and r.prefill_remaining == 1 and r.tokens_fed > 0]
        prefillers = [r for r in self._running if r.pending_row is None and r not in decoders]
        for running in on_device:
            if budget <= 0:
                break
            if len(running.tokens_generated) + 1 >= running.request.max_tokens:
                continue
            entries.append(StepEntry(running.request_id, [0], [0], device_row=running.pending_row))
            owners.append(running)
            budget -= 1
        for running in decoders:
            if budget <= 0:
                break
            entries.append(StepEntry(running.request_id, [running.feed[-1]], [0]))
            owners.append(running)
            budget -= 1
        for running in sorted(prefillers, key=lambda r: r.admitted_order):
            if budget <= 0:
                break
            count = min(self.chunk_size, running.prefill_remaining, budget)
            if count <= 0:
                continue
            feed = running.feed
            portion = feed[running.tokens_fed : running.tokens_fed + count]
            completes = running.tokens_fed + count == len(feed)
            entries.append(StepEntry(running.request_id, portion, [count - 1] if completes else []))
            owners.append(running)
            budget -= count
        return entries, owners

    def _preempt_youngest(self) -> bool:
        """Free the youngest running request and queue it first for recompute.

        Returns False when nothing can be preempted (then the error is real).  A
        request that is alone and still does not fit is finished as "cancelled".
        """
        if not self._running:
            return False
        victim = max(self._running, key=lambda r: r.admitted_order)
        self._running.remove(victim)
        victim.draws = self.cache.states.draws(self.cache.state_slot(victim.request_id))
        self.cache.free_request(victim.request_id)
        if not self._running:
            self.stats["rejected"] += 1
            self._finish(victim, "cancelled", already_freed=True)
            return True
        victim.state = RequestState.WAITING
        victim.tokens_fed = 0
        victim.preemptions += 1
        self.stats["preemptions"] += 1
        with self._lock:
            self._waiting.appendleft(victim)
        return True

    def _accept_token(self, running: RunningRequest, token: int) -> None:
        params = running.request.sampling_params
        if token in self.eos_token_ids and not params.ignore_eos:
            self._finish(running, "stop")
            return
        running.tokens_generated.append(token)
        text = self.tokenizer.decode([token]) if self.tokenizer is not None else ""
        running.steps.append(GenerationStep(text=text, num_tokens=1, tokens=(token,)))
        if len(running.tokens_generated) >= running.request.max_tokens:
            self._finish(running, "length")

    def _finish(self, running: RunningRequest, reason: str, already_freed: bool = False) -> None:
        if running.state == RequestState.DONE:
            return
        running.finish_reason = reason  # type: ignore[assignment]
        running.pending_row = None
        in_cache = running in self._running and not already_freed
        running.state = RequestState.DONE
        if in_cache and self.cache.has_request(running.request_id):
            self.cache.free_request(running.request_id)
        running.steps.append(GenerationStep(text="", finish_reason=reason))  # type: ignore[arg-type]
        running.done_event.set()

    def _reap_done(self) -> None:
        self._running = [r for r in self._running if r.state != RequestState.DONE]

    def _result_of(self, running: RunningRequest) -> GenerationResult:
        tokens = list(running.tokens_generated)
        text = self.tokenizer.decode(tokens) if self.tokenizer is not None else ""
        return GenerationResult(
            text=text,
            tokens=tokens,
            finish_reason=running.finish_reason or "cancelled",
            prompt_tokens=len(running.prompt_token_ids),
        )
