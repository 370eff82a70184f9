"""The cache manager: pages of keys and values with a block table per request,
and slots for per-request state of fixed size.

Entries of the model's execution order that need a cache are put into GROUPS
by what they need (kv heads, head size, window).  A group has one page pool
and one device tensor [entries, 2 (K|V), pages, kv_heads, page_size, head_dim];
a page id is valid in every entry of its group, and each request has one block
table per group.  A windowed group gives a page back as soon as no later query
can see any of its positions; its table entry becomes -1 and is never
addressed again.  All pages of a request go back when it is released.

Beside the pages there are `max_seqs` state slots.  A request holds one slot
from admission to release; mixers with a `StateNeed` get a tensor
[max_seqs, *shape] indexed by the slot, zeroed at admission.

The reference keeps one pool and one table per layer, all identical
(src/llaisys/kv_cache/block_kv_cache.hpp:16-96, src/llaisys/models/qwen2.cpp:832-845)
and frees only when a request ends (:1066-1070).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import torch

from ..parts.base import PagedKVNeed, StateNeed
from .pool import PagePool


class CacheFull(RuntimeError):
    """Not enough free pages (or no free state slot) for what was asked."""


@dataclass
class CacheView:
    """What a mixer sees of the cache for one entry of the execution order."""
    owned: bool                      # False: reads another entry's cache, writes nothing
    group: Optional[int] = None      # index of the page group (paged needs)
    k: Optional[torch.Tensor] = None     # [pages, kv_heads, page_size, head_dim]
    v: Optional[torch.Tensor] = None
    page_size: int = 0
    state: Optional[torch.Tensor] = None  # [max_seqs, *shape] (state needs)


@dataclass
class _Group:
    need: PagedKVNeed
    entries: List[int]
    pool: PagePool
    data: torch.Tensor               # [n_entries, 2, pages, kv_heads, page_size, head_dim]


@dataclass
class _Request:
    slot: int
    cached: int = 0
    tables: List[List[int]] = field(default_factory=list)    # per group: logical block -> page or -1
    first_live: List[int] = field(default_factory=list)      # per group: first block not yet given back


class CacheManager:
    def __init__(self, needs: Sequence[object], sources: Sequence[Optional[int]], *,
                 page_size: int, num_pages: int, max_seqs: int, dtype: torch.dtype,
                 device, page_order_seed: Optional[int] = None):
        """`needs[i]` is what entry i of the execution order needs (None for
        nothing), `sources[i]` the entry whose cache it reads instead of its own.
        `num_pages` is the number of pages of EVERY group."""
        if page_size <= 0:
            raise ValueError("cache: page_size must be positive")
        self.page_size = int(page_size)
        self.max_seqs = int(max_seqs)
        self.device = torch.device(device)
        self.groups: List[_Group] = []
        self._entry_group: Dict[int, Tuple[int, int]] = {}     # entry -> (group, index in group)
        self._entry_state: Dict[int, torch.Tensor] = {}
        self._sources = list(sources)
        by_need: Dict[PagedKVNeed, int] = {}
        for i, need in enumerate(needs):
            if sources[i] is not None or need is None:
                continue
            if isinstance(need, PagedKVNeed):
                if need not in by_need:
                    by_need[need] = len(self.groups)
                    self.groups.append(_Group(need, [], None, None))
                g = by_need[need]
                self._entry_group[i] = (g, len(self.groups[g].entries))
                self.groups[g].entries.append(i)
            elif isinstance(need, StateNeed):
                self._entry_state[i] = torch.zeros((self.max_seqs, *need.shape), dtype=need.dtype,
                                                   device=self.device)
            else:
                raise TypeError(f"cache: entry {i} has an unknown cache need {need!r}")
        for gi, g in enumerate(self.groups):
            order = None
            if page_order_seed is not None:
                gen = torch.Generator().manual_seed(page_order_seed + gi)
                order = torch.randperm(num_pages, generator=gen).tolist()
            g.pool = PagePool(num_pages, order)
            g.data = torch.zeros((len(g.entries), 2, num_pages, g.need.num_kv_heads, self.page_size,
                                  g.need.head_dim), dtype=dtype, device=self.device)
        self._free_slots = list(range(self.max_seqs))[::-1]
        self._requests: Dict[Hashable, _Request] = {}

    # ---- views ---------------------------------------------------------
    def view(self, entry: int) -> CacheView:
        src = self._sources[entry]
        owner = entry if src is None else src
        if owner in self._entry_group:
            g, j = self._entry_group[owner]
            d = self.groups[g].data
            return CacheView(owned=src is None, group=g, k=d[j, 0], v=d[j, 1], page_size=self.page_size)
        if owner in self._entry_state:
            return CacheView(owned=src is None, state=self._entry_state[owner])
        return CacheView(owned=src is None)

    # ---- requests --------------------------------------------------------
    def has(self, rid) -> bool:
        return rid in self._requests

    def live(self) -> List[Hashable]:
        return list(self._requests)

    def free_slots(self) -> int:
        return len(self._free_slots)

    def free_pages(self) -> List[int]:
        return [g.pool.free for g in self.groups]

    def admit(self, rid) -> int:
        if rid in self._requests:
            raise KeyError(f"cache: request {rid!r} is already live")
        if not self._free_slots:
            raise CacheFull(f"cache: all {self.max_seqs} state slots are taken")
        slot = self._free_slots.pop()
        self._requests[rid] = _Request(slot, 0, [[] for _ in self.groups], [0 for _ in self.groups])
        for st in self._entry_state.values():
            st[slot].zero_()
        return slot

    def slot(self, rid) -> int:
        return self._requests[rid].slot

    def cached_len(self, rid) -> int:
        return self._requests[rid].cached

    def block_table(self, rid, group: int) -> List[int]:
        return self._requests[rid].tables[group]

    def _first_needed_block(self, g: _Group, first_query_pos: int) -> int:
        """First block that a query at `first_query_pos` or later can see."""
        if g.need.window <= 0:
            return 0
        return max(0, first_query_pos - g.need.window + 1) // self.page_size

    def pages_needed(self, rid, n_new: int, cached: Optional[int] = None) -> List[int]:
        """Pages each group must take so that `n_new` more tokens of `rid` fit
        (rid may be unknown: then it is counted as a new request)."""
        r = self._requests.get(rid)
        have_cached = (r.cached if r is not None else 0) if cached is None else cached
        out = []
        for gi, g in enumerate(self.groups):
            nblk = -(-(have_cached + n_new) // self.page_size)
            have = len(r.tables[gi]) if r is not None else 0
            out.append(max(0, nblk - have))
        return out

    def reserve(self, rid, n_new: int) -> None:
        """Take the pages that positions cached..cached+n_new-1 need, in every
        group, or none at all (CacheFull)."""
        r = self._requests[rid]
        need = self.pages_needed(rid, n_new)
        for g, n in zip(self.groups, need):
            if n > g.pool.free:
                raise CacheFull(f"cache: request {rid!r} needs {n} more pages, "
                                f"{g.pool.free} of {g.pool.capacity} are free")
        for gi, (g, n) in enumerate(zip(self.groups, need)):
            for _ in range(n):
                r.tables[gi].append(g.pool.alloc())

    def commit(self, rid, n_new: int) -> None:
        """`n_new` tokens were written: advance, and give back the pages that
        the window has passed."""
        r = self._requests[rid]
        r.cached += n_new
        for gi, g in enumerate(self.groups):
            if g.need.window <= 0:
                continue
            keep_from = self._first_needed_block(g, r.cached)
            for b in range(r.first_live[gi], min(keep_from, len(r.tables[gi]))):
                if r.tables[gi][b] >= 0:
                    g.pool.release(r.tables[gi][b])
                    r.tables[gi][b] = -1
            r.first_live[gi] = max(r.first_live[gi], min(keep_from, len(r.tables[gi])))

    def release(self, rid) -> None:
        r = self._requests.pop(rid)
        for gi, g in enumerate(self.groups):
            for p in r.tables[gi]:
                if p >= 0:
                    g.pool.release(p)
        self._free_slots.append(r.slot)

    def check_invariants(self) -> None:
        """No page lost, held twice or on the free list while in a table."""
        for gi, g in enumerate(self.groups):
            seen = {}
            for rid, r in self._requests.items():
                for p in r.tables[gi]:
                    if p < 0:
                        continue
                    if p in seen:
                        raise AssertionError(f"page {p} of group {gi} is held by {seen[p]!r} and {rid!r}")
                    if not g.pool.is_held(p):
                        raise AssertionError(f"page {p} of group {gi} is in a table but free")
                    seen[p] = rid
            if len(seen) != g.pool.used:
                raise AssertionError(f"group {gi}: {g.pool.used} pages taken, {len(seen)} in tables")
        slots = [r.slot for r in self._requests.values()]
        if len(set(slots)) != len(slots) or set(slots) & set(self._free_slots):
            raise AssertionError("state slots are held twice or free while held")
        if len(slots) + len(self._free_slots) != self.max_seqs:
            raise AssertionError("state slots lost")
