"""Slots for per-request state of fixed size.

Beside the paged keys and values, a request owns one row in each state tensor
for as long as it lives: `[max_requests, *shape]` per layer call that asked for
state.  A row is zeroed when it is handed out.  The reference keeps such state
in a separate cache family (cache/state_cache.py:130-333); here it lives next to
the pages so one manager admits and frees a request as a whole.  Llama needs no
state tensors; the slot itself (the row index) still exists for every request.
"""

from __future__ import annotations

import torch

from mini_infer_amd.exceptions import OutOfMemoryError
from mini_infer_amd.parts.base import StateNeeds


class StateSlots:
    def __init__(
        self,
        max_requests: int,
        needs: dict[int, StateNeeds],
        device,
        allocate_storage: bool = True,
    ) -> None:
        if max_requests <= 0:
            raise ValueError(f"max_requests must be positive, got {max_requests}")
        self.max_requests = max_requests
        self._free: list[int] = list(range(max_requests - 1, -1, -1))
        self._owner: list[object | None] = [None] * max_requests
        self.tensors: dict[int, torch.Tensor] = {}
        if allocate_storage:
            for call, need in needs.items():
                self.tensors[call] = torch.zeros((max_requests, *need.shape), dtype=need.dtype, device=device)

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self, owner: object) -> int:
        if not self._free:
            raise OutOfMemoryError(f"all {self.max_requests} request slots are in use")
        slot = self._free.pop()
        self._owner[slot] = owner
        for tensor in self.tensors.values():
            tensor[slot].zero_()
        return slot

    def free(self, slot: int) -> None:
        if not 0 <= slot < self.max_requests:
            raise ValueError(f"slot {slot} is outside 0..{self.max_requests - 1}")
        if self._owner[slot] is None:
            raise RuntimeError(f"state slot {slot} freed twice (or never allocated)")
        self._owner[slot] = None
        self._free.append(slot)

    def owner(self, slot: int) -> object | None:
        return self._owner[slot]

    def check(self) -> None:
        if len(set(self._free)) != len(self._free):
            raise AssertionError("a state slot is in the free list twice")
        held = sum(owner is not None for owner in self._owner)
        if held + len(self._free) != self.max_requests:
            raise AssertionError("a state slot is lost")
        for slot in self._free:
            if self._owner[slot] is not None:
                raise AssertionError(f"state slot {slot} is both free and owned")
