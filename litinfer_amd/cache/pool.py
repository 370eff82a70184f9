"""A pool of page ids with a free list (kept by the host library, csrc/host.cpp).

The reference's pool (src/llaisys/kv_cache/block_kv_cache.hpp:16-63) is a LIFO
list per layer without a guard; here one id is valid for every layer of a
group, and taking a page twice or giving one back twice is an error.
"""
from __future__ import annotations

from typing import Iterable, Optional

from . import native


class PagePoolError(RuntimeError):
    pass


class PagePool:
    def __init__(self, num_pages: int, order: Optional[Iterable[int]] = None, _borrowed=None):
        self._lib = native.lib()
        self._owned = _borrowed is None
        if _borrowed is not None:                      # a group's pool inside a cache manager's book
            self._p = _borrowed
            return
        ids = None if order is None else [int(i) for i in order]
        if ids is not None and len(ids) != int(num_pages):
            raise ValueError("page pool: the free-list order must be a permutation of all page ids")
        self._p = self._lib.li_pool_create(int(num_pages), native.int_array(ids) if ids is not None else None)
        if self.capacity == 0:
            msg = self._lib.li_pool_error(self._p).decode()
            self._lib.li_pool_destroy(self._p)
            self._p = None
            raise ValueError(msg)

    def __del__(self):
        if getattr(self, "_owned", False) and getattr(self, "_p", None):
            self._lib.li_pool_destroy(self._p)
            self._p = None

    def _fail(self):
        raise PagePoolError(self._lib.li_pool_error(self._p).decode())

    @property
    def capacity(self) -> int:
        return self._lib.li_pool_capacity(self._p)

    @property
    def free(self) -> int:
        return self._lib.li_pool_free(self._p)

    @property
    def used(self) -> int:
        return self.capacity - self.free

    @property
    def total_allocations(self) -> int:
        return self._lib.li_pool_total_allocations(self._p)

    @property
    def peak_used(self) -> int:
        """The most pages that were held at one time so far."""
        return self._lib.li_pool_peak_used(self._p)

    def alloc(self) -> int:
        p = self._lib.li_pool_alloc(self._p)
        if p < 0:
            self._fail()
        return p

    def release(self, page: int) -> None:
        if self._lib.li_pool_release(self._p, int(page)) < 0:
            self._fail()

    def is_held(self, page: int) -> bool:
        return bool(self._lib.li_pool_is_held(self._p, int(page)))
