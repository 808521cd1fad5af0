"""Decode steps replayed as HIP graphs.

A decode step (one token per request) launches some three hundred small kernels;
issued one by one from Python their launch cost exceeds their run time at small
batches.  Such a step is captured once per (batch bucket, block-table width) and
replayed: per step the host then only fills one staging buffer, copies it, and
launches the graph.  The reference does the same with CUDA graphs per batch
bucket (engine/paged_decode_graph.py:42-225: buckets 1..32, padding rows write to
a scratch block); here padding rows write nowhere (slot -1).

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


def bucket_of(value: int, minimum: int = 1) -> int:
    bucket = minimum
    while bucket < value:
        bucket *= 2
    return bucket


class DecodeGraph:
    """One captured decode step for `batch` rows and block tables `width` pages wide."""

    def __init__(self, runner, batch: int, width: int, max_device_tokens: int = 64) -> None:
        self.runner = runner
        self.batch = batch
        self.width = width
        self.num_groups = len(runner.cache.groups)
        # layout of the staging buffer (all int32): see `fill`
        b = batch
        self.sizes = [b, b, b, b + 1, b, b, b] + [n for _ in range(self.num_groups) for n in (b, b * width)] + [b]
        self.total = sum(self.sizes)
        self.host = torch.empty(self.total, dtype=torch.int32, pin_memory=True)
        self.device = torch.zeros(self.total, dtype=torch.int32, device=runner.device)
        views = list(torch.split(self.device, self.sizes))
        slot_mapping = [views[7 + 2 * g] for g in range(self.num_groups)]
        block_tables = [views[8 + 2 * g].view(batch, width) for g in range(self.num_groups)]
        # rows whose token is still on the device take it from `device_tokens` (first node of the graph)
        self.from_rows = views[-1]
        self.device_tokens = torch.zeros(max_device_tokens, dtype=torch.int32, device=runner.device)
        cu = list(range(batch + 1))
        self.ctx = StepContext(
            num_tokens=batch,
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
            max_q_len=1,
            max_seq_len=width * runner.block_size,
            host_cu_seqlens_q=cu,
            host_seq_lens=[1] * batch,
            host_state_slots=[0] * batch,
        )
        self.graph: torch.cuda.CUDAGraph | None = None
        self.real = 0  # rows of the staged step that belong to requests
        self.logits: torch.Tensor | None = None
        self._copied: torch.cuda.Event | None = None  # set once the staging buffer may be rewritten

    def fill(self, token_ids: np.ndarray, index, from_rows: np.ndarray | None = None) -> None:
        """Write this step's integers (padded to the bucket) into the pinned staging buffer."""
        b, real = self.batch, len(index.request_ids)
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

        put(token_ids, b)
        put(index.positions, b)
        put(np.arange(b, dtype=np.int32), b)  # token_request: one token per row
        put(np.arange(b + 1, dtype=np.int32), b + 1)  # cu_seqlens_q
        put(index.seq_lens, b, pad=1)
        put(index.state_slots, b, pad=-1)  # padding rows own no state slot
        put(np.arange(b, dtype=np.int32), b)  # logits wanted at every row
        for mapping, table in zip(index.slot_mapping, index.block_tables):
            put(mapping, b, pad=-1)  # padding rows write no keys or values
            wide = host[at : at + b * self.width].reshape(b, self.width)
            wide[:real, : table.shape[1]] = table
            wide[:real, table.shape[1] :] = -1
            at += b * self.width
        put(from_rows if from_rows is not None else np.empty(0, dtype=np.int32), b, pad=-1)
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
        # No garbage collection while the stream records: a collector run frees whatever cyclic
        # garbage earlier work left (pinned buffers, events, other graphs), their destructors make
        # runtime calls that a recording stream forbids, and an error inside a destructor aborts.
        collecting = gc.isenabled()
        gc.collect()
        gc.disable()
        try:
            with torch.cuda.graph(graph):
                ops.begin_step(self.ctx.token_ids, self.from_rows, self.device_tokens, self.runner.vocab_size,
                               self.runner.cache.states.table, self.ctx.state_slots, self.ctx.seq_lens)
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
    ) -> torch.Tensor:
        """Send this step's integers to the device; returns the state-slot id of each real row
        (on the device, valid in stream order from here on, until the next `stage`)."""
        self.fill(token_ids, index, from_rows)
        self.device.copy_(self.host, non_blocking=True)
        if from_rows is not None and device_tokens is not None:
            self.device_tokens[: device_tokens.numel()].copy_(device_tokens, non_blocking=True)
        if self._copied is None:
            self._copied = torch.cuda.Event()
        self._copied.record()
        self.real = len(index.request_ids)
        return self.ctx.state_slots[: self.real]

    def replay(self) -> tuple[torch.Tensor, torch.Tensor]:
        """Run the staged step.  Logits [real rows, vocab] and the state-slot id of each row;
        both live until the next replay."""
        if self.graph is None:
            self.capture()
        self.graph.replay()
        return self.logits[: self.real], self.ctx.state_slots[: self.real]


class DecodeGraphs:
    """The captured steps of one runner, by (batch bucket, width bucket)."""

    def __init__(self, runner, max_batch: int = 64) -> None:
        self.runner = runner
        self.max_batch = max_batch
        self.graphs: dict[tuple[int, int], DecodeGraph] = {}
        self.replays = 0

    def takes(self, index, rows: np.ndarray, device_tokens: torch.Tensor | None = None) -> bool:
        real = len(index.request_ids)
        return (
            index.max_q_len == 1
            and real <= self.max_batch
            and len(rows) == real
            and bool((rows == np.arange(real)).all())
            and (device_tokens is None or device_tokens.numel() <= self.max_batch)
        )

    def stage(
        self,
        token_ids: np.ndarray,
        index,
        from_rows: np.ndarray | None = None,
        device_tokens: torch.Tensor | None = None,
    ) -> tuple[DecodeGraph, torch.Tensor]:
        """The recorded step that takes this batch, its integers sent to the device, and the
        state-slot ids of its rows; `graph.replay()` then runs it."""
        batch = bucket_of(len(index.request_ids))
        width = bucket_of(max([t.shape[1] for t in index.block_tables] + [1]), MIN_WIDTH)
        key = (batch, width)
        graph = self.graphs.get(key)
        if graph is None:
            graph = self.graphs[key] = DecodeGraph(self.runner, batch, width, self.max_batch)
        self.replays += 1
        return graph, graph.stage(token_ids, index, from_rows, device_tokens)
