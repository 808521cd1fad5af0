"""The runner: a loaded model, its cache, and the one step function.

`ModelRunner.from_pretrained` mirrors the reference's constructor of the same
name (engine/model_runner.py:84-175: model folder, `dtype`, `num_blocks`,
`block_size`).  `step` is the single primitive (the reference's
`forward_step_packed`, engine/model_runner.py:270-395): a flattened batch of
prompt portions beside single decoded tokens, run from the cache, returning
logits only at the wanted places.
"""

from __future__ import annotations

from pathlib import Path
from typing import Any, Hashable, Sequence

import numpy as np
import torch

from mini_infer_amd import ops
from mini_infer_amd.cache.manager import CacheManager
from mini_infer_amd.config import DEFAULT_BLOCK_SIZE, DEFAULT_NUM_BLOCKS, EngineConfig, read_config_json
from mini_infer_amd.engine.batch import StepEntry
from mini_infer_amd.engine.decode_graph import DecodeGraphs
from mini_infer_amd.models import architecture_for
from mini_infer_amd.parts.base import StepContext
from mini_infer_amd.weights import load_checkpoint
from mini_infer_amd.weights.random_init import fill_random_on_device

_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}
# Steps of single tokens are recorded up to this many requests (in buckets of powers of two).  At
# the widths of a 3B model a step of 128 single tokens keeps the device busy for about as long as
# the host needs to launch it kernel by kernel; beyond 256 the device is the slower of the two.
MAX_RECORDED_BATCH = 256


def resolve_dtype(dtype: str | torch.dtype | None) -> torch.dtype:
    if dtype is None:
        return torch.bfloat16
    if isinstance(dtype, torch.dtype):
        if dtype not in _DTYPES.values():
            raise ValueError(f"dtype must be bfloat16 or float32, got {dtype}")
        return dtype
    if dtype not in _DTYPES:
        raise ValueError(f"dtype must be one of {sorted(_DTYPES)}, got {dtype!r}")
    return _DTYPES[dtype]


def require_gpu(device: str | torch.device) -> torch.device:
    device = torch.device(device)
    if device.type != "cuda" or not torch.cuda.is_available():
        raise RuntimeError(
            "mini_infer_amd runs on an AMD GPU through its HIP kernels; there is no CPU path "
            f"(asked for {device}, torch.cuda.is_available()={torch.cuda.is_available()})"
        )
    return device


class ModelRunner:
    def __init__(
        self,
        model: Any,
        config: Any,
        *,
        num_blocks: int = DEFAULT_NUM_BLOCKS,
        block_size: int = DEFAULT_BLOCK_SIZE,
        max_concurrent: int = 16,
        cuda_graph: bool = True,
    ) -> None:
        self.model = model
        self.config = config
        self.dtype = model.dtype
        self.device = model.device
        self.vocab_size = model.vocab_size
        # the most positions a request may reach, if the model says (admission goes by it)
        self.max_model_len: int | None = getattr(model, "max_position_embeddings", None)
        self.block_size = block_size
        self.num_blocks = num_blocks
        self.cache = CacheManager(
            model.cache_needs(block_size),
            page_size=block_size,
            num_pages=num_blocks,
            max_requests=max_concurrent,
            dtype=model.dtype,
            device=model.device,
        )
        self._layer_caches = self.cache.layer_caches()
        self.engine_config: EngineConfig | None = None  # set when built from one
        # state-slot id of every row of the logits the last step returned (int32, on the device)
        self.last_row_slots: torch.Tensor | None = None
        # small steps (single tokens, and few tokens with portions among them) are replayed as HIP
        # graphs where every part of the model allows it
        self.decode_graphs = DecodeGraphs(self, max_batch=MAX_RECORDED_BATCH) if cuda_graph and model.graph_safe else None

    # -- construction -----------------------------------------------------------

    @classmethod
    def from_pretrained(
        cls,
        model_name: str | Path,
        *,
        engine: EngineConfig | None = None,
        device: str = "cuda:0",
        dtype: str | torch.dtype | None = None,
        num_blocks: int = DEFAULT_NUM_BLOCKS,
        block_size: int = DEFAULT_BLOCK_SIZE,
        max_concurrent: int = 16,
        cuda_graph: bool = True,
    ) -> "ModelRunner":
        """Load the model folder `model_name` (config.json + safetensors) and build its cache.

        The engine's knobs come as one `EngineConfig` (`engine=`) or as the keyword arguments
        of the same names, from which one is made (and so checked) here."""
        if engine is None:
            engine = EngineConfig(
                num_blocks=num_blocks, block_size=block_size, max_concurrent=max_concurrent, device=device,
                dtype=str(resolve_dtype(dtype)).replace("torch.", ""), cuda_graph=cuda_graph,
            )
        dev = require_gpu(engine.device)
        raw = read_config_json(model_name)
        arch = architecture_for(raw)
        config = arch.parse_config(raw)
        model = arch.make_model(config, resolve_dtype(engine.dtype), dev)
        load_checkpoint(model, model_name)
        runner = cls(model, config, num_blocks=engine.num_blocks, block_size=engine.block_size,
                     max_concurrent=engine.max_concurrent, cuda_graph=engine.cuda_graph)
        runner.engine_config = engine
        return runner

    @classmethod
    def from_random(
        cls,
        raw_config: dict[str, Any],
        seed: int,
        *,
        device: str = "cuda:0",
        dtype: str | torch.dtype | None = None,
        num_blocks: int = DEFAULT_NUM_BLOCKS,
        block_size: int = DEFAULT_BLOCK_SIZE,
        max_concurrent: int = 16,
        std: float = 0.02,
        norm_jitter: float = 0.0,
        cuda_graph: bool = True,
    ) -> "ModelRunner":
        """Random weights made on the device (no file): for sizes too large to write out."""
        dev = require_gpu(device)
        arch = architecture_for(raw_config)
        config = arch.parse_config(raw_config)
        model = arch.make_model(config, resolve_dtype(dtype), dev)
        fill_random_on_device(model, seed, std=std, norm_jitter=norm_jitter)
        return cls(model, config, num_blocks=num_blocks, block_size=block_size, max_concurrent=max_concurrent,
                   cuda_graph=cuda_graph)

    supports_device_tokens = True  # `step(entries, device_tokens=)`, `StepEntry.device_row`

    # -- requests ---------------------------------------------------------------

    def add_request(self, request_id: Hashable) -> None:
        self.cache.add_request(request_id)

    def has_request(self, request_id: Hashable) -> bool:
        return self.cache.has_request(request_id)

    def free_request(self, request_id: Hashable) -> None:
        self.cache.free_request(request_id)

    def num_free_blocks(self) -> int:
        """Free pages of the fullest page group; all `num_blocks` for a model that keeps no
        pages at all (state of fixed size only), which seats alone then bound."""
        if not self.cache.groups:
            return self.num_blocks
        return min(self.cache.num_free_pages(g.index) for g in self.cache.groups)

    # -- the step ---------------------------------------------------------------

    def step(self, entries: Sequence[StepEntry], device_tokens: torch.Tensor | None = None) -> torch.Tensor:
        """Run the given tokens as one batch from the cache; logits [wanted, vocab] float32.

        Rows come in the order of `entries` and, within an entry, of its `want`.
        The tensor may be reused by the next step: read or copy it before calling
        `step` again.  Requests seen for the first time are admitted.  Raises `OutOfMemoryError`
        before anything changes if the pages for this step are not there; any other failure
        (a kernel that refuses a size, an error on the device) gives the step's pages back
        and forgets the requests it admitted, so lengths and free pages are what they were;
        where the model keeps state of fixed size, the rows of the step's requests are copied
        aside before the forward pass and put back, so a mixer that had already updated them in
        place leaves no trace either.

        `device_tokens` (int32, on the device) holds token ids the host has not read yet,
        e.g. what `sample_tokens` returned for the last step; an entry with `device_row`
        takes its token from there, so the next step can be launched before the ids of the
        last one have come back (the reference's asynchronous sampling,
        scheduler/continuous_scheduler.py:529-646).
        """
        entries = [e for e in entries if len(e.tokens) > 0]
        if not entries:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=self.device)
        seen: set[Hashable] = set()
        for entry in entries:
            if entry.request_id in seen:
                raise ValueError(f"request {entry.request_id!r} appears twice in one step")
            seen.add(entry.request_id)
            for w in entry.want:
                if not 0 <= w < len(entry.tokens):
                    raise ValueError(
                        f"request {entry.request_id!r}: wanted place {w} is outside its {len(entry.tokens)} tokens"
                    )
        token_ids = np.concatenate([np.asarray(e.tokens, dtype=np.int64) for e in entries])
        if token_ids.min() < 0 or token_ids.max() >= self.vocab_size:
            raise ValueError(f"token ids must lie in 0..{self.vocab_size - 1}")
        from_rows: np.ndarray | None = None
        if any(e.device_row is not None for e in entries):
            if device_tokens is None or device_tokens.dtype != torch.int32 or device_tokens.dim() != 1:
                raise ValueError("entries with device_row need device_tokens, a 1-d int32 tensor on the device")
            from_rows = np.full(token_ids.size, -1, dtype=np.int32)
            at = 0
            for entry in entries:
                if entry.device_row is not None:
                    if len(entry.tokens) != 1 or not 0 <= entry.device_row < device_tokens.numel():
                        raise ValueError(
                            f"request {entry.request_id!r}: device_row goes with exactly one placeholder token "
                            f"and must index the {device_tokens.numel()} device tokens"
                        )
                    from_rows[at] = entry.device_row
                at += len(entry.tokens)

        admitted: list[Hashable] = []
        try:
            for entry in entries:
                if not self.cache.has_request(entry.request_id):
                    self.cache.add_request(entry.request_id)
                    admitted.append(entry.request_id)
            extents = {e.request_id: len(e.tokens) for e in entries}
            self.cache.reserve(extents)
        except Exception:
            for request_id in admitted:
                self.cache.free_request(request_id)
            raise

        # From here on pages are reserved: whatever fails below (building the index, the copy
        # to the device, a kernel that refuses a size) gives them back, so that the cache is
        # as it was before the step (the reference's rollback on a failed step:
        # scheduler/continuous_scheduler.py:418-445).  Keys and values the failed step may
        # have written lie past every request's length and are overwritten later.
        states = self.cache.states
        saved: tuple[torch.Tensor, list[torch.Tensor]] | None = None
        try:
            index = self.cache.build_step_index([(e.request_id, len(e.tokens)) for e in entries])
            rows = np.fromiter(
                (int(index.cu_seqlens_q[b]) + w for b, e in enumerate(entries) for w in e.want),
                dtype=np.int32,
            )
            token_ids = token_ids.astype(np.int32)
            states.flush()  # slot-table rows of requests admitted since the last step
            if self.decode_graphs is not None and self.decode_graphs.takes(index, rows, device_tokens):
                graph, step_slots = self.decode_graphs.stage(token_ids, index, from_rows, device_tokens)
                if states.has_state:
                    saved = (step_slots, states.snapshot(step_slots))
                logits, self.last_row_slots = graph.replay()
            elif self.decode_graphs is not None and self.decode_graphs.takes_mixed(index, [e.want for e in entries], device_tokens):
                graph, step_slots = self.decode_graphs.stage_mixed(
                    token_ids, index, [e.want for e in entries], from_rows, device_tokens
                )
                if states.has_state:
                    saved = (step_slots, states.snapshot(step_slots))
                logits, self.last_row_slots = graph.replay()
            else:
                row_slots = np.fromiter(
                    (index.state_slots[b] for b, e in enumerate(entries) for _ in e.want), dtype=np.int32
                )
                ctx, from_rows_device, self.last_row_slots = self._to_device(token_ids, rows, index, from_rows, row_slots)
                if states.has_state:
                    saved = (ctx.state_slots, states.snapshot(ctx.state_slots))
                # tokens still on the device are taken from there, positions go into the state slots
                if self.device.type == "cuda":
                    ops.begin_step(ctx.token_ids, from_rows_device, device_tokens, self.vocab_size,
                                   states.table, ctx.state_slots, ctx.seq_lens)
                logits = self.model.forward(ctx, self._layer_caches)
        except BaseException:
            # the host's books first (nothing here touches the device), then what the device holds:
            # if the device itself is what failed, that part may fail again, and the first
            # error is the one to report
            self.cache.cancel_reservation(extents, push=False)
            for request_id in admitted:
                extents.pop(request_id, None)
                self.cache.free_request(request_id)
            try:
                if saved is not None:
                    states.restore(*saved)
                self.cache.push_positions(extents)
            except Exception:  # noqa: BLE001
                pass
            raise
        self.cache.commit(extents)
        return logits

    def _to_device(
        self, token_ids: np.ndarray, rows: np.ndarray, index, from_rows: np.ndarray | None, row_slots: np.ndarray
    ) -> tuple[StepContext, torch.Tensor | None, torch.Tensor]:
        """All of a step's integers in one pinned buffer and one copy to the device
        (the step's context, `from_rows` on the device if it was given, and `row_slots`)."""
        pieces = [
            token_ids,
            index.positions,
            index.token_request,
            index.cu_seqlens_q,
            index.seq_lens,
            index.state_slots,
            rows,
            row_slots,
        ]
        for mapping, table in zip(index.slot_mapping, index.block_tables):
            pieces.append(mapping)
            pieces.append(table.reshape(-1))
        if from_rows is not None:
            pieces.append(from_rows)
        sizes = [int(p.size) for p in pieces]
        staging = torch.empty(sum(sizes), dtype=torch.int32, pin_memory=self.device.type == "cuda")
        host = staging.numpy()
        offset = 0
        for piece, size in zip(pieces, sizes):
            host[offset : offset + size] = piece
            offset += size
        on_device = staging.to(self.device, non_blocking=True)
        views = list(torch.split(on_device, sizes))
        token_ids_d, positions, token_request, cu, seq_lens, state_slots, rows_d, row_slots_d = views[:8]
        slot_mapping, block_tables = [], []
        for g, table in enumerate(index.block_tables):
            slot_mapping.append(views[8 + 2 * g])
            block_tables.append(views[9 + 2 * g].view(table.shape))
        ctx = StepContext(
            num_tokens=int(token_ids.size),
            num_requests=len(index.request_ids),
            page_size=self.block_size,
            token_ids=token_ids_d,
            positions=positions,
            token_request=token_request,
            cu_seqlens_q=cu,
            seq_lens=seq_lens,
            state_slots=state_slots,
            logit_rows=rows_d,
            slot_mapping=slot_mapping,
            block_tables=block_tables,
            max_q_len=index.max_q_len,
            max_seq_len=index.max_seq_len,
            host_cu_seqlens_q=index.cu_seqlens_q.tolist(),
            host_seq_lens=index.seq_lens.tolist(),
            host_state_slots=index.state_slots.tolist(),
        )
        return ctx, (views[-1] if from_rows is not None else None), row_slots_d
