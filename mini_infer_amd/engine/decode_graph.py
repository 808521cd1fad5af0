"""Small steps replayed as HIP graphs.

A decode step (one token per request) launches some three hundred small kernels;
issued one by one from Python their launch cost exceeds their run time at small
batches, and so does that of any step of a few dozen tokens (4-5 ms of host time for 32
layers against a millisecond or two on the device).  Such steps are captured once per
bucket and replayed: per step the host then only fills one staging buffer, copies it, and
launches the graph.  The reference does the same with CUDA graphs, per batch bucket for
decode steps (engine/paged_decode_graph.py:42-225: buckets 1..32, padding rows write to a
scratch block) and per (tokens, requests) bucket for steps with portions of prompts in them
(engine/paged_prefill_graph.py:104-120); here padding rows write nowhere (slot -1).

Two kinds of recorded step:
  * single tokens: `batch` requests with one token each, bucketed by (batch, block-table
    width); the request boundaries are the same in every replay;
  * mixed: up to `tokens` tokens of up to `requests` requests, portions of prompts beside single
    tokens in any division, bucketed by (tokens, requests, width).  The boundaries differ
    from replay to replay, so they live on the device only (`StepContext.host_*` are None) and
    every launch is shaped by the bucket alone.  Tokens past the real ones belong to one
    more request that owns no page and no state slot; requests past that one bring no token.
    Logits are computed at one row per request (its wanted row, or its first for a request
    that wants none) and the wanted ones are picked out afterwards.

Only models whose parts declare `graph_safe` are captured: a part that loops on
the host over `ctx.host_*` lists cannot be replayed with other lengths.
"""

from __future__ import annotations

import gc

import numpy as np
import torch

from mini_infer_amd import ops
from mini_infer_amd.parts.base import StepContext

MIN_WIDTH = 16
MIXED_MIN_TOKENS = 16
# A step of more tokens than this keeps the device busy for longer than the host needs to launch it
# (at the widths of a 1B model; at 8B widths that already holds from a few dozen tokens on, and
# recording only frees the host).  Measured, 16 prompts of 16 tokens in one step, time to the first
# token recorded / kernel by kernel: 2.8 / 4.0 ms at 1B widths, 5.5 / 5.6 at 3B, 8.7 / 8.5 at 8B;
# a 16-token prompt beside 8 single tokens: 2.9 / 3.8 ms at 3B, 4.6 / 4.4 at 8B.
MIXED_MAX_TOKENS = 256


def bucket_of(value: int, minimum: int = 1) -> int:
    bucket = minimum
    while bucket < value:
        bucket *= 2
    return bucket


class DecodeGraph:
    """One captured step: `batch` requests and `tokens` tokens (`tokens == batch` and one token
    each for a single-token step, `mixed` otherwise), block tables `width` pages wide."""

    def __init__(self, runner, batch: int, width: int, max_device_tokens: int = 64, tokens: int | None = None) -> None:
        self.runner = runner
        self.batch = batch
        self.width = width
        self.mixed = tokens is not None
        self.tokens = t = batch if tokens is None else tokens
        self.num_groups = len(runner.cache.groups)
        # layout of the staging buffer (all int32): see `fill`
        b = batch
        self.sizes = [t, t, t, b + 1, b, b, b] + [n for _ in range(self.num_groups) for n in (t, b * width)] + [t, b]
        self.total = sum(self.sizes)
        self.host = torch.empty(self.total, dtype=torch.int32, pin_memory=True)
        self.device = torch.zeros(self.total, dtype=torch.int32, device=runner.device)
        views = list(torch.split(self.device, self.sizes))
        slot_mapping = [views[7 + 2 * g] for g in range(self.num_groups)]
        block_tables = [views[8 + 2 * g].view(batch, width) for g in range(self.num_groups)]
        # rows whose token is still on the device take it from `device_tokens` (first node of the graph)
        self.from_rows = views[-2]
        self.pick_from = views[-1]  # mixed steps: the requests whose logits were asked for, in order
        self.device_tokens = torch.zeros(max_device_tokens, dtype=torch.int32, device=runner.device)
        self.ctx = StepContext(
            num_tokens=t,
            num_requests=batch,
            page_size=runner.block_size,
            token_ids=views[0],
            positions=views[1],
            token_request=views[2],
            cu_seqlens_q=views[3],
            seq_lens=views[4],
            state_slots=views[5],
            logit_rows=views[6],
            slot_mapping=slot_mapping,
            block_tables=block_tables,
            max_q_len=t if self.mixed else 1,
            max_seq_len=width * runner.block_size,
            # single tokens: the boundaries of every replay; mixed: known on the device only
            host_cu_seqlens_q=None if self.mixed else list(range(batch + 1)),
            host_seq_lens=None if self.mixed else [1] * batch,
            host_state_slots=None if self.mixed else [0] * batch,
        )
        self.graph: torch.cuda.CUDAGraph | None = None
        self.real = 0  # requests of the staged step (single tokens: its rows)
        self.picked: torch.Tensor | None = None  # mixed: rows of `logits` that were asked for
        self.logits: torch.Tensor | None = None
        self._copied: torch.cuda.Event | None = None  # set once the staging buffer may be rewritten

    def fill(self, token_ids: np.ndarray, index, from_rows: np.ndarray | None = None,
             wanted_row: np.ndarray | None = None) -> None:
        """Write this step's integers (padded to the bucket) into the pinned staging buffer.
        `wanted_row[b]` (mixed steps): the token row whose logits request b wants, or -1."""
        b, t, real = self.batch, self.tokens, len(index.request_ids)
        real_tokens = int(token_ids.size)
        if self._copied is not None:
            self._copied.synchronize()  # the last step's copy out of this buffer is done
        host = self.host.numpy()
        host[:] = 0
        at = 0

        def put(values: np.ndarray, size: int, pad: int = 0) -> None:
            nonlocal at
            host[at : at + len(values)] = values
            if pad and len(values) < size:
                host[at + len(values) : at + size] = pad
            at += size

        put(token_ids, t)
        if not self.mixed:
            put(index.positions, b)
            put(np.arange(b, dtype=np.int32), b)  # token_request: one token per row
            put(np.arange(b + 1, dtype=np.int32), b + 1)  # cu_seqlens_q
            put(index.seq_lens, b, pad=1)
            put(index.state_slots, b, pad=-1)  # padding rows own no state slot
            put(np.arange(b, dtype=np.int32), b)  # logits wanted at every row
        else:
            # the tokens past the real ones are those of one more request, at positions 0, 1, ...;
            # the requests after it bring nothing
            spare = t - real_tokens
            assert real < b or spare == 0
            host[at : at + real_tokens] = index.positions
            host[at + real_tokens : at + t] = np.arange(spare, dtype=np.int32)
            at += t
            host[at : at + real_tokens] = index.token_request
            host[at + real_tokens : at + t] = real
            at += t
            host[at : at + real + 1] = index.cu_seqlens_q
            host[at + real + 1 : at + b + 1] = t
            at += b + 1
            put(index.seq_lens, b, pad=1)
            if real < b:
                host[at - b + real] = max(spare, 1)
            put(index.state_slots, b, pad=-1)
            rows = np.where(wanted_row >= 0, wanted_row, index.cu_seqlens_q[:-1]).astype(np.int32)
            put(rows, b)  # (requests past the real ones: row 0, whose logits nobody reads)
        for mapping, table in zip(index.slot_mapping, index.block_tables):
            put(mapping, t, pad=-1)  # padding rows write no keys or values
            wide = host[at : at + b * self.width].reshape(b, self.width)
            wide[:real, : table.shape[1]] = table
            wide[:real, table.shape[1] :] = -1
            at += b * self.width
        put(from_rows if from_rows is not None else np.empty(0, dtype=np.int32), t, pad=-1)
        put(np.flatnonzero(wanted_row >= 0).astype(np.int32) if wanted_row is not None else np.empty(0, dtype=np.int32), b)
        assert at == self.total

    def capture(self) -> None:
        """Run once outside a graph (library handles, workspaces), then record.

        The run outside the graph must leave no trace, since the replay that follows does the
        step's work again: keys and values land in the same places both times, and per-request
        state is kept out of it by giving every row slot -1 (the state tensors' spare row)
        for that run.
        """
        model, caches = self.runner.model, self.runner._layer_caches
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            self.ctx.shared.clear()
            slots = self.ctx.state_slots.clone()
            self.ctx.state_slots.fill_(-1)
            model.forward(self.ctx, caches)
            self.ctx.state_slots.copy_(slots)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.ctx.shared.clear()
        graph = torch.cuda.CUDAGraph()
        table = self.runner.cache.states.table  # (whatever is still to be sent to it goes now, not into the recording)
        # No garbage collection while the stream records: a collector run frees whatever cyclic
        # garbage earlier work left (pinned buffers, events, other graphs), their destructors make
        # runtime calls that a recording stream forbids, and an error inside a destructor aborts.
        collecting = gc.isenabled()
        gc.collect()
        gc.disable()
        try:
            with torch.cuda.graph(graph):
                ops.begin_step(self.ctx.token_ids, self.from_rows, self.device_tokens, self.runner.vocab_size,
                               table, self.ctx.state_slots, self.ctx.seq_lens)
                self.logits = model.forward(self.ctx, caches)
        finally:
            if collecting:
                gc.enable()
        self.graph = graph

    def stage(
        self,
        token_ids: np.ndarray,
        index,
        from_rows: np.ndarray | None = None,
        device_tokens: torch.Tensor | None = None,
        wanted_row: np.ndarray | None = None,
    ) -> torch.Tensor:
        """Send this step's integers to the device; returns the state-slot id of each real request
        (on the device, valid in stream order from here on, until the next `stage`)."""
        self.fill(token_ids, index, from_rows, wanted_row)
        self.device.copy_(self.host, non_blocking=True)
        if from_rows is not None and device_tokens is not None:
            self.device_tokens[: device_tokens.numel()].copy_(device_tokens, non_blocking=True)
        if self._copied is None:
            self._copied = torch.cuda.Event()
        self._copied.record()
        self.real = len(index.request_ids)
        self.picked = None
        if self.mixed and not bool((wanted_row >= 0).all()):
            self.picked = self.pick_from[: int((wanted_row >= 0).sum())]
        return self.ctx.state_slots[: self.real]

    def replay(self) -> tuple[torch.Tensor, torch.Tensor]:
        """Run the staged step.  Logits [wanted rows, vocab] and the state-slot id of each of
        them; both live until the next replay."""
        if self.graph is None:
            self.capture()
        self.graph.replay()
        if self.picked is not None:
            return self.logits.index_select(0, self.picked), self.ctx.state_slots.index_select(0, self.picked)
        return self.logits[: self.real], self.ctx.state_slots[: self.real]


class DecodeGraphs:
    """The captured steps of one runner: single-token steps by (batch bucket, width bucket),
    mixed ones by (token bucket, request bucket, width bucket)."""

    def __init__(self, runner, max_batch: int = 64, mixed: bool = True) -> None:
        self.runner = runner
        self.max_batch = max_batch
        self.mixed = mixed
        self.graphs: dict[tuple[int, ...], DecodeGraph] = {}
        self.replays = 0
        self.mixed_replays = 0

    def takes(self, index, rows: np.ndarray, device_tokens: torch.Tensor | None = None) -> bool:
        """Whether a step of single tokens, logits wanted at every row, is replayed."""
        real = len(index.request_ids)
        return (
            index.max_q_len == 1
            and real <= self.max_batch
            and len(rows) == real
            and bool((rows == np.arange(real)).all())
            and (device_tokens is None or device_tokens.numel() <= self.max_batch)
        )

    def takes_mixed(self, index, wants: list, device_tokens: torch.Tensor | None = None) -> bool:
        """Whether a step that is not one of single tokens with every row wanted is replayed: few
        tokens, at most one wanted row a request."""
        total = int(index.cu_seqlens_q[-1])
        return (
            self.mixed
            and total <= MIXED_MAX_TOKENS
            and all(len(w) <= 1 for w in wants)
            and (device_tokens is None or device_tokens.numel() <= self.max_batch)
        )

    def stage(
        self,
        token_ids: np.ndarray,
        index,
        from_rows: np.ndarray | None = None,
        device_tokens: torch.Tensor | None = None,
    ) -> tuple[DecodeGraph, torch.Tensor]:
        """The recorded step that takes this batch of single tokens, its integers sent to the
        device, and the state-slot ids of its rows; `graph.replay()` then runs it."""
        batch = bucket_of(len(index.request_ids))
        width = bucket_of(max([t.shape[1] for t in index.block_tables] + [1]), MIN_WIDTH)
        key = (batch, width)
        graph = self.graphs.get(key)
        if graph is None:
            graph = self.graphs[key] = DecodeGraph(self.runner, batch, width, self.max_batch)
        self.replays += 1
        return graph, graph.stage(token_ids, index, from_rows, device_tokens)

    def stage_mixed(
        self,
        token_ids: np.ndarray,
        index,
        wants: list,
        from_rows: np.ndarray | None = None,
        device_tokens: torch.Tensor | None = None,
    ) -> tuple[DecodeGraph, torch.Tensor]:
        """The same for a step with portions in it; `wants[b]` holds request b's wanted place among
        its own tokens, or nothing."""
        real = len(index.request_ids)
        tokens = bucket_of(int(token_ids.size), MIXED_MIN_TOKENS)
        # (one request more than the real ones where tokens are left over: the one they belong to)
        batch = bucket_of(real + (1 if tokens > token_ids.size else 0))
        width = bucket_of(max([t.shape[1] for t in index.block_tables] + [1]), MIN_WIDTH)
        key = (tokens, batch, width)
        graph = self.graphs.get(key)
        if graph is None:
            graph = self.graphs[key] = DecodeGraph(self.runner, batch, width, self.max_batch, tokens=tokens)
        wanted_row = np.fromiter(
            (int(index.cu_seqlens_q[b]) + w[0] if len(w) else -1 for b, w in enumerate(wants)), dtype=np.int64, count=real
        )
        self.mixed_replays += 1
        return graph, graph.stage(token_ids, index, from_rows, device_tokens, wanted_row)
