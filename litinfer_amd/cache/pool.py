"""A pool of page ids with a free list.

The reference's pool (src/llaisys/kv_cache/block_kv_cache.hpp:16-63) is a LIFO
list per layer without a guard; here one id is valid for every layer of a
group, and taking a page twice or giving one back twice is an error.
"""
from __future__ import annotations

from typing import Iterable, List, Optional


class PagePoolError(RuntimeError):
    pass


class PagePool:
    def __init__(self, num_pages: int, order: Optional[Iterable[int]] = None):
        if num_pages <= 0:
            raise ValueError(f"page pool: needs at least one page, found {num_pages}")
        self.capacity = int(num_pages)
        ids = list(range(self.capacity)) if order is None else [int(i) for i in order]
        if sorted(ids) != list(range(self.capacity)):
            raise ValueError("page pool: the free-list order must be a permutation of all page ids")
        self._free: List[int] = ids[::-1]          # alloc() pops from the end: first id of `order` first
        self._held = [False] * self.capacity
        self.total_allocations = 0

    @property
    def free(self) -> int:
        return len(self._free)

    @property
    def used(self) -> int:
        return self.capacity - len(self._free)

    def alloc(self) -> int:
        if not self._free:
            raise PagePoolError("page pool: no free page")
        p = self._free.pop()
        if self._held[p]:
            raise PagePoolError(f"page pool: page {p} was on the free list while held")
        self._held[p] = True
        self.total_allocations += 1
        return p

    def release(self, page: int) -> None:
        if not 0 <= page < self.capacity:
            raise PagePoolError(f"page pool: page id {page} out of range")
        if not self._held[page]:
            raise PagePoolError(f"page pool: page {page} freed twice")
        self._held[page] = False
        self._free.append(page)

    def is_held(self, page: int) -> bool:
        return self._held[page]
