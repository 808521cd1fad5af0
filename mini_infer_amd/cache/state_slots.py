"""Slots for per-request state of fixed size.

Beside the paged keys and values, a request owns one slot for as long as it lives.
The reference keeps such state in a separate cache family
(cache/state_cache.py:130-333); here it lives next to the pages so one manager
admits and frees a request as a whole.  A slot is

  * one row of the *slot table*, `[max_requests, 8]` int32 on the device with a copy
    on the host: the request's position (tokens in the cache) and the state of its
    sampling (seed, index of the next draw, temperature, top-k, top-p).  Kernels
    read a request's row by its slot id: the sampling kernel takes its settings
    from there and advances the draw index itself, the first kernel of a step
    writes the positions.  The host copy is what the scheduler plans with; both
    are advanced by the same events, so they agree whenever the device is idle;
  * one row in each state tensor a mixer asked for, `[max_requests + 1, *shape]` per
    layer call (several per call, each of its own shape and dtype, where the mixer named
    several), zeroed when the slot is handed out (Llama asks for none).  The last
    row belongs to no request: the padding rows of a recorded decode step carry slot
    -1, which indexes it, so a mixer that reads and writes `state[slots]` with device
    tensors alone needs no special case for them and can be recorded.

Rows of the slot table travel to the device through a small ring of pinned staging rows
and asynchronous copies (a copy from pageable memory would wait for the stream to drain,
and an admission would cost the overlap that sampling ahead of the host is there for).
The zeroed row of a slot just handed out waits for the sampling settings that usually follow
(`set_sampling` sends the row, once) or for the device's next need of the table (`table`).
"""

from __future__ import annotations

import numpy as np
import torch

from mini_infer_amd.exceptions import OutOfMemoryError
from mini_infer_amd.parts.base import StateNeeds

# int32 words of a slot-table row (the layout the kernels read)
SLOT_WORDS = 8
SLOT_POSITION = 0
SLOT_SEED_LO = 1
SLOT_SEED_HI = 2
SLOT_DRAW = 3
SLOT_TEMPERATURE = 4  # float32 bits
SLOT_TOP_K = 5
SLOT_TOP_P = 6  # float32 bits


def _float_bits(value: float) -> int:
    return int(np.array([value], dtype=np.float32).view(np.int32)[0])


def _as_i32(value: int) -> int:
    """The int32 holding the unsigned 32-bit pattern `value`."""
    return int(np.array([value & 0xFFFFFFFF], dtype=np.uint32).view(np.int32)[0])


STAGING_ROWS = 64  # pinned rows a slot-table row waits in for its copy to the device


class StateSlots:
    def __init__(
        self,
        max_requests: int,
        needs: "dict[int, StateNeeds | dict[str, StateNeeds]]",
        device,
        allocate_storage: bool = True,
    ) -> None:
        if max_requests <= 0:
            raise ValueError(f"max_requests must be positive, got {max_requests}")
        self.max_requests = max_requests
        self._free: list[int] = list(range(max_requests - 1, -1, -1))
        self._owner: list[object | None] = [None] * max_requests
        # per layer call: the one tensor it asked for, or its tensors by name
        self.tensors: "dict[int, torch.Tensor | dict[str, torch.Tensor]]" = {}
        self._all_tensors: list[torch.Tensor] = []
        self.host = np.zeros((max_requests, SLOT_WORDS), dtype=np.int32)
        self._table: torch.Tensor | None = None
        self._dirty: set[int] = set()  # rows whose host copy the device has not been sent yet
        self._staging: torch.Tensor | None = None
        self._staging_events: list = []
        self._staging_at = 0
        # whether any layer call keeps state of its own (with or without storage to put it in)
        self.has_state = bool(needs)
        if allocate_storage:
            device = torch.device(device)
            self._table = torch.zeros((max_requests, SLOT_WORDS), dtype=torch.int32, device=device)
            if device.type == "cuda":
                self._staging = torch.empty((STAGING_ROWS, SLOT_WORDS), dtype=torch.int32, pin_memory=True)
                self._staging_events = [None] * STAGING_ROWS

            def make(need: StateNeeds) -> torch.Tensor:
                tensor = torch.zeros((max_requests + 1, *need.shape), dtype=need.dtype, device=device)
                self._all_tensors.append(tensor)
                return tensor

            for call, need in needs.items():
                if isinstance(need, StateNeeds):
                    self.tensors[call] = make(need)
                else:
                    self.tensors[call] = {name: make(one) for name, one in need.items()}

    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def table(self) -> torch.Tensor | None:
        """The slot table on the device, every row changed on the host since sent first."""
        self.flush()
        return self._table

    def allocate(self, owner: object) -> int:
        """A free slot, its table row and state rows zeroed: position 0, draw 0, greedy."""
        if not self._free:
            raise OutOfMemoryError(f"all {self.max_requests} request slots are in use")
        slot = self._free.pop()
        self._owner[slot] = owner
        self.host[slot] = 0
        self.host[slot, SLOT_TOP_P] = _float_bits(1.0)
        self._dirty.add(slot)
        for tensor in self._all_tensors:
            tensor[slot].zero_()
        return slot

    # -- state rows of a step, kept aside and put back ------------------------------------

    def snapshot(self, slots: torch.Tensor) -> list[torch.Tensor]:
        """Copies of the state rows of `slots` (int64 or int32 indices on the device, -1 for
        nobody's row), one per state tensor: what `restore` puts back when the step that was
        about to update them fails."""
        index = slots.long()
        return [tensor.index_select(0, torch.where(index < 0, index + tensor.shape[0], index)) for tensor in self._all_tensors]

    def restore(self, slots: torch.Tensor, saved: list[torch.Tensor]) -> None:
        index = slots.long()
        for tensor, rows in zip(self._all_tensors, saved):
            tensor.index_copy_(0, torch.where(index < 0, index + tensor.shape[0], index), rows)

    def free(self, slot: int) -> None:
        if not 0 <= slot < self.max_requests:
            raise ValueError(f"slot {slot} is outside 0..{self.max_requests - 1}")
        if self._owner[slot] is None:
            raise RuntimeError(f"state slot {slot} freed twice (or never allocated)")
        self._owner[slot] = None
        self._free.append(slot)

    def owner(self, slot: int) -> object | None:
        return self._owner[slot]

    # -- the slot table -----------------------------------------------------------

    def _send(self, slot: int, words: slice) -> None:
        """Queue the copy of `host[slot, words]` to the device, ordered after the work already
        queued; the values are those of this moment (they wait in a pinned row of their own)."""
        if self._table is None:
            return
        values = torch.from_numpy(self.host[slot, words].copy())
        if self._staging is None:
            self._table[slot, words].copy_(values)
            return
        at = self._staging_at
        self._staging_at = (at + 1) % STAGING_ROWS
        if self._staging_events[at] is not None:
            self._staging_events[at].synchronize()  # the copy that last used this row is done
        else:
            self._staging_events[at] = torch.cuda.Event()
        row = self._staging[at, words]
        row.copy_(values)
        self._table[slot, words].copy_(row, non_blocking=True)
        self._staging_events[at].record()

    def push(self, slot: int) -> None:
        """Send the host's copy of a whole row to the device now."""
        self._dirty.discard(slot)
        self._send(slot, slice(0, SLOT_WORDS))

    def push_position(self, slot: int) -> None:
        """Send the host's position of a slot alone: what a step that did not happen, or tokens
        that were taken back, leave to put right.  The other words are the device's to keep
        (it advances the draw index itself)."""
        if slot in self._dirty:
            return  # the whole row is still to be sent, position included
        self._send(slot, slice(SLOT_POSITION, SLOT_POSITION + 1))

    def flush(self) -> None:
        """Send every row changed on the host since it was last sent."""
        for slot in sorted(self._dirty):
            self._send(slot, slice(0, SLOT_WORDS))
        self._dirty.clear()

    def set_sampling(
        self, slot: int, *, temperature: float, top_k: int, top_p: float, seed: int, draw: int = 0
    ) -> None:
        """The sampling state of the request in `slot`: its settings, its seed (64 unsigned
        bits) and the index of its next draw (0 for a new request, the number of tokens it
        already drew when it is admitted again after a preemption)."""
        row = self.host[slot]
        row[SLOT_SEED_LO] = _as_i32(seed)
        row[SLOT_SEED_HI] = _as_i32(seed >> 32)
        row[SLOT_DRAW] = _as_i32(draw)
        row[SLOT_TEMPERATURE] = _float_bits(temperature)
        row[SLOT_TOP_K] = int(top_k)
        row[SLOT_TOP_P] = _float_bits(top_p)
        self.push(slot)  # (with the zeroed row of `allocate`, if that is still waiting: one copy)

    def set_position(self, slot: int, position: int) -> None:
        """Host copy only: on the device the first kernel of the step writes the same value."""
        self.host[slot, SLOT_POSITION] = position

    def count_draw(self, slot: int) -> None:
        """Host copy only: the sampling kernel advances the device's copy itself."""
        self.host[slot, SLOT_DRAW] = _as_i32(int(self.host[slot, SLOT_DRAW]) + 1)

    def position(self, slot: int) -> int:
        return int(self.host[slot, SLOT_POSITION])

    def draws(self, slot: int) -> int:
        return int(self.host[slot, SLOT_DRAW]) & 0xFFFFFFFF

    def seed(self, slot: int) -> int:
        lo = int(self.host[slot, SLOT_SEED_LO]) & 0xFFFFFFFF
        hi = int(self.host[slot, SLOT_SEED_HI]) & 0xFFFFFFFF
        return (hi << 32) | lo

    # -- checks ---------------------------------------------------------------------

    def check(self) -> None:
        if len(set(self._free)) != len(self._free):
            raise AssertionError("a state slot is in the free list twice")
        held = sum(owner is not None for owner in self._owner)
        if held + len(self._free) != self.max_requests:
            raise AssertionError("a state slot is lost")
        for slot in self._free:
            if self._owner[slot] is not None:
                raise AssertionError(f"state slot {slot} is both free and owned")
