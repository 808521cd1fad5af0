"""The cache manager: pages of keys and values, block tables, state slots.

Layer calls whose needs agree (same key/value heads, key and value widths, window
and value layout) form a *group*.  Each group has its own page storage, its own pool of page ids and,
per request, its own block table; pages are shared by all calls of the group
(one id addresses the same page in every call's storage, as the reference's
block ids are global across layers: cache/block_pool.py:338-351).

Life of a request:
  add_request      takes a state slot
  reserve          before a step: pages for the new tokens of ALL requests of the
                   step, all or nothing (no partial growth to roll back, unlike
                   the reference's per-slot growth: cache/paged_kv_cache.py:716-734)
  commit           after the step: lengths advance; a windowed group gives back
                   the pages no future query can see
  free_request     every page and the state slot go back; ids are reused at once

Storage per group: keys [calls, num_pages, kv_heads, page_size * head_dim] and values
[calls, num_pages, kv_heads, page_size * value dim], sized apart (a mixer may keep
values of another width than its keys, or none).  A key chunk is
[page_size][head_dim]; a value chunk is [page_size][value dim], or transposed
([value dim][page_size]) if the mixer that reads it asked for that layout.
"""

from __future__ import annotations

import dataclasses
from typing import Hashable

import numpy as np
import torch

from mini_infer_amd.cache.page_pool import PagePool
from mini_infer_amd.cache.state_slots import StateSlots
from mini_infer_amd.exceptions import OutOfMemoryError
from mini_infer_amd.parts.base import CacheNeeds, LayerCache, StateNeeds

RELEASED = -1  # block-table entry of a page a window has passed


@dataclasses.dataclass
class PageGroup:
    index: int
    calls: list[int]
    num_kv_heads: int
    head_dim: int
    window: int | None
    pool: PagePool
    value_dim: int = 0  # width of a value row; 0: the group keeps no values
    v_transposed: bool = False  # values stored [dim][slot] inside a page, as its mixers asked
    k_storage: torch.Tensor | None = None
    v_storage: torch.Tensor | None = None
    tables: dict[Hashable, list[int]] = dataclasses.field(default_factory=dict)

    def first_live_page(self, length: int, page_size: int) -> int:
        """Index of the first page a query at position `length` (or later) can see."""
        if self.window is None:
            return 0
        return max(0, length - self.window + 1) // page_size


@dataclasses.dataclass
class StepIndex:
    """Host arrays describing one step, ready to be copied to the device."""

    request_ids: list[Hashable]
    token_request: np.ndarray  # [T] batch row of each token
    positions: np.ndarray  # [T]
    cu_seqlens_q: np.ndarray  # [B+1]
    seq_lens: np.ndarray  # [B] length after the step
    state_slots: np.ndarray  # [B]
    slot_mapping: list[np.ndarray]  # per group [T]
    block_tables: list[np.ndarray]  # per group [B, max_blocks]
    max_q_len: int
    max_seq_len: int


class CacheManager:
    def __init__(
        self,
        needs: list[CacheNeeds | None],
        *,
        page_size: int,
        num_pages: int,
        max_requests: int,
        dtype: torch.dtype = torch.float32,
        device="cpu",
        allocate_storage: bool = True,
    ) -> None:
        if page_size <= 0:
            raise ValueError(f"page_size must be positive, got {page_size}")
        self.page_size = page_size
        self.num_pages = num_pages
        self.dtype = dtype
        self.device = torch.device(device)
        self.groups: list[PageGroup] = []
        self._group_of_call: dict[int, int] = {}
        by_shape: dict[tuple, PageGroup] = {}
        state_needs: "dict[int, StateNeeds | dict[str, StateNeeds]]" = {}
        for call, need in enumerate(needs):
            if need is None:
                continue
            if need.pages is not None:
                pages = need.pages
                if pages.num_kv_heads <= 0 or pages.head_dim <= 0 or pages.value_dim < 0:
                    raise ValueError(f"call {call}: impossible page needs {pages}")
                key = (pages.num_kv_heads, pages.head_dim, pages.value_dim, pages.window, pages.v_transposed)
                group = by_shape.get(key)
                if group is None:
                    group = PageGroup(
                        index=len(self.groups),
                        calls=[],
                        num_kv_heads=pages.num_kv_heads,
                        head_dim=pages.head_dim,
                        window=pages.window,
                        pool=PagePool(num_pages),
                        value_dim=pages.value_dim,
                        v_transposed=pages.v_transposed,
                    )
                    by_shape[key] = group
                    self.groups.append(group)
                group.calls.append(call)
                self._group_of_call[call] = group.index
            if need.state is not None:
                if isinstance(need.state, StateNeeds):
                    state_needs[call] = need.state
                else:
                    named = dict(need.state)
                    if not named or not all(isinstance(k, str) and isinstance(v, StateNeeds) for k, v in named.items()):
                        raise ValueError(f"call {call}: state needs are one StateNeeds or a non-empty mapping of names to them")
                    state_needs[call] = named
        for group in self.groups:
            if allocate_storage:
                calls, heads = len(group.calls), group.num_kv_heads
                group.k_storage = torch.zeros(
                    (calls, num_pages, heads, page_size * group.head_dim), dtype=dtype, device=self.device
                )
                if group.value_dim > 0:
                    group.v_storage = torch.zeros(
                        (calls, num_pages, heads, page_size * group.value_dim), dtype=dtype, device=self.device
                    )
        self.states = StateSlots(max_requests, state_needs, self.device, allocate_storage)
        self._num_calls = len(needs)
        self._lengths: dict[Hashable, int] = {}
        self._slots: dict[Hashable, int] = {}

    # -- requests -----------------------------------------------------------

    def add_request(self, request_id: Hashable) -> int:
        if request_id in self._lengths:
            raise ValueError(f"request {request_id!r} is already in the cache")
        slot = self.states.allocate(request_id)
        self._lengths[request_id] = 0
        self._slots[request_id] = slot
        for group in self.groups:
            group.tables[request_id] = []
        return slot

    def has_request(self, request_id: Hashable) -> bool:
        return request_id in self._lengths

    def length(self, request_id: Hashable) -> int:
        return self._lengths[request_id]

    def state_slot(self, request_id: Hashable) -> int:
        return self._slots[request_id]

    def set_sampling(self, request_id: Hashable, *, temperature: float, top_k: int, top_p: float,
                     seed: int, draw: int = 0) -> None:
        """Write the request's sampling state into its slot (see `StateSlots.set_sampling`)."""
        self.states.set_sampling(self._slots[request_id], temperature=temperature, top_k=top_k, top_p=top_p,
                                 seed=seed, draw=draw)

    def live_requests(self) -> list[Hashable]:
        return list(self._lengths)

    def free_request(self, request_id: Hashable) -> None:
        if request_id not in self._lengths:
            raise KeyError(f"request {request_id!r} is not in the cache")
        for group in self.groups:
            for page in group.tables.pop(request_id):
                if page != RELEASED:
                    group.pool.free(page)
        self.states.free(self._slots.pop(request_id))
        del self._lengths[request_id]

    # -- pages --------------------------------------------------------------

    @property
    def has_pages(self) -> bool:
        """Whether any layer call keeps keys and values in pages (a model of state mixers
        alone has none, and then no page count bounds what it can hold)."""
        return bool(self.groups)

    def num_free_pages(self, group: int = 0) -> int:
        return self.groups[group].pool.num_free

    def pages_needed(self, request_id: Hashable, new_tokens: int) -> list[int]:
        """Pages each group must add for `new_tokens` more tokens of the request."""
        length = self._lengths[request_id]
        total = -(-(length + new_tokens) // self.page_size)
        return [max(0, total - len(group.tables[request_id])) for group in self.groups]

    def pages_for_tokens(self, tokens: int) -> int:
        return -(-tokens // self.page_size) if self.groups else 0

    def reserve(self, extents: dict[Hashable, int]) -> None:
        """Pages for all `request -> new tokens` of a step, or `OutOfMemoryError` and no change."""
        wanted = [0] * len(self.groups)
        for request_id, new_tokens in extents.items():
            if new_tokens < 0:
                raise ValueError(f"request {request_id!r}: negative token count {new_tokens}")
            for g, count in enumerate(self.pages_needed(request_id, new_tokens)):
                wanted[g] += count
        for group, count in zip(self.groups, wanted):
            if count > group.pool.num_free:
                raise OutOfMemoryError(
                    f"page group {group.index} needs {count} more pages, {group.pool.num_free} "
                    f"of {group.pool.num_pages} are free"
                )
        for request_id, new_tokens in extents.items():
            for group, count in zip(self.groups, self.pages_needed(request_id, new_tokens)):
                group.tables[request_id].extend(group.pool.allocate_many(count))

    def cancel_reservation(self, extents: dict[Hashable, int], push: bool = True) -> None:
        """Undo a `reserve` whose step did not happen: pages past what each request's
        committed length needs go back; lengths were never advanced.  All of the host's books
        are put right first; only then (`push`) are the positions sent to the device again,
        which the step's first kernel may already have overwritten (`push_positions`)."""
        for request_id in extents:
            keep = self.pages_for_tokens(self._lengths[request_id])
            for group in self.groups:
                table = group.tables[request_id]
                while len(table) > keep:
                    page = table.pop()
                    if page != RELEASED:
                        group.pool.free(page)
        if push:
            self.push_positions(extents)

    def push_positions(self, request_ids) -> None:
        """Send the host's position of each of these requests to its slot on the device."""
        for request_id in request_ids:
            if request_id in self._slots:
                self.states.push_position(self._slots[request_id])

    def commit(self, extents: dict[Hashable, int]) -> None:
        """Advance lengths after a step and give back what windows have passed."""
        for request_id, new_tokens in extents.items():
            length = self._lengths[request_id] + new_tokens
            self._lengths[request_id] = length
            self.states.set_position(self._slots[request_id], length)
            for group in self.groups:
                if group.window is None:
                    continue
                table = group.tables[request_id]
                for i in range(min(group.first_live_page(length, self.page_size), len(table))):
                    if table[i] != RELEASED:
                        group.pool.free(table[i])
                        table[i] = RELEASED

    def truncate(self, request_id: Hashable, length: int) -> None:
        """Forget tokens past `length`; whole pages past it go back (the partial one stays).

        The reference's `truncate_to` (cache/paged_kv_cache.py:260-306).  A
        windowed group cannot be truncated below what it has already released.
        """
        if not 0 <= length <= self._lengths[request_id]:
            raise ValueError(f"cannot truncate {request_id!r} from {self._lengths[request_id]} to {length}")
        keep = self.pages_for_tokens(length)
        for group in self.groups:
            table = group.tables[request_id]
            if group.window is not None and any(
                p == RELEASED for p in table[group.first_live_page(length, self.page_size) : keep]
            ):
                raise ValueError("a windowed group has already released pages this truncation needs")
            while len(table) > keep:
                page = table.pop()
                if page != RELEASED:
                    group.pool.free(page)
        self._lengths[request_id] = length
        self.states.set_position(self._slots[request_id], length)
        self.states.push_position(self._slots[request_id])

    # -- per-step index -------------------------------------------------------

    def build_step_index(self, entries: list[tuple[Hashable, int]]) -> StepIndex:
        """Host arrays for a step of `(request, new tokens)` entries, in that order.

        Call after `reserve`.  Positions continue each request's length; slot
        mappings address the reserved pages.
        """
        num_requests = len(entries)
        q_lens = np.fromiter((n for _, n in entries), dtype=np.int64, count=num_requests)
        starts = np.fromiter((self._lengths[r] for r, _ in entries), dtype=np.int64, count=num_requests)
        cu = np.zeros(num_requests + 1, dtype=np.int32)
        np.cumsum(q_lens, out=cu[1:])
        total = int(cu[-1])
        token_request = np.repeat(np.arange(num_requests, dtype=np.int32), q_lens)
        positions = (np.arange(total, dtype=np.int64) - np.repeat(cu[:-1].astype(np.int64), q_lens)
                     + np.repeat(starts, q_lens)).astype(np.int32)
        seq_lens = (starts + q_lens).astype(np.int32)
        slots = np.fromiter((self._slots[r] for r, _ in entries), dtype=np.int32, count=num_requests)
        slot_mapping: list[np.ndarray] = []
        block_tables: list[np.ndarray] = []
        for group in self.groups:
            width = max([len(group.tables[r]) for r, _ in entries] + [1])
            table = np.full((num_requests, width), RELEASED, dtype=np.int32)
            for b, (request_id, _) in enumerate(entries):
                pages = group.tables[request_id]
                table[b, : len(pages)] = pages
            page_of_token = table[token_request, positions // self.page_size].astype(np.int64)
            mapping = page_of_token * self.page_size + positions % self.page_size
            if total and (page_of_token < 0).any():
                raise AssertionError("a token of this step would be written to a released page")
            slot_mapping.append(mapping.astype(np.int32))
            block_tables.append(table)
        return StepIndex(
            request_ids=[r for r, _ in entries],
            token_request=token_request,
            positions=positions,
            cu_seqlens_q=cu,
            seq_lens=seq_lens,
            state_slots=slots,
            slot_mapping=slot_mapping,
            block_tables=block_tables,
            max_q_len=int(q_lens.max()) if num_requests else 0,
            max_seq_len=int(seq_lens.max()) if num_requests else 0,
        )

    # -- views for the model --------------------------------------------------

    def layer_caches(self) -> list[LayerCache]:
        """One `LayerCache` per layer call (empty for calls that own no cache)."""
        caches = [LayerCache() for _ in range(self._num_calls)]
        for group in self.groups:
            for i, call in enumerate(group.calls):
                caches[call].group = group.index
                caches[call].v_transposed = group.v_transposed
                pages, heads = self.num_pages, group.num_kv_heads
                if group.k_storage is not None:
                    caches[call].k_pages = group.k_storage[i].view(pages, heads, self.page_size, group.head_dim)
                if group.v_storage is not None:
                    shape = (group.value_dim, self.page_size) if group.v_transposed else (self.page_size, group.value_dim)
                    caches[call].v_pages = group.v_storage[i].view(pages, heads, *shape)
        for call, tensor in self.states.tensors.items():
            caches[call].state = tensor
        return caches

    # -- checks -----------------------------------------------------------------

    def check(self) -> None:
        """No page lost, held twice or freed twice; tables agree with the pools."""
        self.states.check()
        for group in self.groups:
            group.pool.check()
            seen: set[int] = set()
            for request_id, table in group.tables.items():
                if request_id not in self._lengths:
                    raise AssertionError(f"group {group.index} has a table for unknown {request_id!r}")
                for page in table:
                    if page == RELEASED:
                        continue
                    if page in seen:
                        raise AssertionError(f"page {page} of group {group.index} is held twice")
                    seen.add(page)
                needed = self.pages_for_tokens(self._lengths[request_id])
                if len(table) < needed:
                    raise AssertionError(f"request {request_id!r} holds fewer pages than its length needs")
            if seen != group.pool.held_pages():
                raise AssertionError(f"group {group.index}: tables and pool disagree about held pages")
