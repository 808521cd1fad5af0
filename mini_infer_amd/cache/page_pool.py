"""A pool of page ids: a free list with checks.

The reference's `BlockPool` keeps a LIFO free list and raises `OutOfMemoryError`
when it is empty (cache/block_pool.py:570-575, :735-757) but does not notice a
double free; this pool does, and can prove that no page is lost or held twice.
"""

from __future__ import annotations

import random

from mini_infer_amd.exceptions import OutOfMemoryError


class PagePool:
    def __init__(self, num_pages: int) -> None:
        if num_pages <= 0:
            raise ValueError(f"num_pages must be positive, got {num_pages}")
        self.num_pages = num_pages
        # LIFO: the page freed last is handed out first, so reuse happens at once.
        # A fresh pool hands its ids out in a scattered order (always the same one for a pool
        # size): requests that grow side by side would otherwise hold neighbouring pages, page j
        # of every request in one small stretch of memory, and a decode step reads page j of all
        # requests at about the same time.  Measured on MI355X at 64 requests: the attention
        # kernel alone runs 21 % slower over pages interleaved that way than over scattered
        # ones (105 against 86 us at 2,100 keys, 197 against 162 us at 4,096), a whole decode
        # step 4 % slower.
        self._free: list[int] = list(range(num_pages))
        random.Random(num_pages).shuffle(self._free)
        self._held = [False] * num_pages

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self) -> int:
        if not self._free:
            raise OutOfMemoryError(f"no free page left (all {self.num_pages} are held)")
        page = self._free.pop()
        self._held[page] = True
        return page

    def allocate_many(self, count: int) -> list[int]:
        """`count` pages or none: raises without taking any if fewer are free."""
        if count > len(self._free):
            raise OutOfMemoryError(f"{count} pages wanted, {len(self._free)} of {self.num_pages} free")
        return [self.allocate() for _ in range(count)]

    def free(self, page: int) -> None:
        if not 0 <= page < self.num_pages:
            raise ValueError(f"page {page} is outside the pool of {self.num_pages}")
        if not self._held[page]:
            raise RuntimeError(f"page {page} freed twice (or never allocated)")
        self._held[page] = False
        self._free.append(page)

    def held_pages(self) -> set[int]:
        return {i for i, held in enumerate(self._held) if held}

    def check(self) -> None:
        """Every page is either free once or held, never both, never neither."""
        free = self._free
        if len(set(free)) != len(free):
            raise AssertionError("a page is in the free list twice")
        for page in free:
            if self._held[page]:
                raise AssertionError(f"page {page} is both free and held")
        if len(free) + sum(self._held) != self.num_pages:
            raise AssertionError("a page is lost: neither free nor held")
