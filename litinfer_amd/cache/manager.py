"""The cache manager: pages of keys and values with a block table per request,
and slots for per-request state of fixed size.

Entries of the model's execution order that need a cache are put into GROUPS
by what they need: the named tensors they keep per token (keys and values of
some head layout, a compressed latent, keys alone ...) and the window.  A
group has one page pool and, for each of its tensors, one device tensor
[entries, pages, *leading sizes, page_size, last size]; a page id is valid in
every entry and every tensor of its group, and each request has one block table
per group.  A windowed group gives a page back as soon as no later query
can see any of its positions; its table entry becomes -1 and is never
addressed again.  All pages of a request go back when it is released.

Beside the pages there are `max_seqs` state slots.  A request holds one slot
from admission to release; mixers with a `StateNeed` get a tensor
[max_seqs, *shape] indexed by the slot, zeroed at admission.  An entry may
need both: one paged need and any number of named states (its view then has
`tensors` and `state`/`states`).

Every group's pool has its own number of pages: a windowed group holds a few
pages a request whatever the context, so it can be far smaller than a group
that keeps all keys.

The bookkeeping itself (pools, tables, slots, the window's give-back) is done by
the host library in C++ (csrc/host.cpp); this class owns the device tensors,
maps request names to the library's handles and turns its codes into exceptions.

The reference keeps one pool and one table per layer, all identical
(src/llaisys/kv_cache/block_kv_cache.hpp:16-96, src/llaisys/models/qwen2.cpp:832-845)
and frees only when a request ends (:1066-1070).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import ctypes

import numpy as np
import torch

from ..parts.base import PagedNeed, StateNeed, needs_of
from . import native
from .pool import PagePool, PagePoolError


class CacheFull(RuntimeError):
    """Not enough free pages (or no free state slot) for what was asked."""


@dataclass
class CacheView:
    """What a mixer sees of the cache for one entry of the execution order."""
    owned: bool                      # False: reads another entry's cache, writes nothing
    group: Optional[int] = None      # index of the page group (paged needs)
    tensors: Optional[Dict[str, torch.Tensor]] = None    # name -> [pages, *leading sizes, page_size, last size]
    page_size: int = 0
    state: Optional[torch.Tensor] = None  # [max_seqs, *shape]: the entry's state (its first, if it has several)
    states: Optional[Dict[str, torch.Tensor]] = None     # name -> [max_seqs, *shape], all of them

    @property
    def k(self) -> Optional[torch.Tensor]:
        """The tensor named "k" (keys [pages, kv_heads, page_size, head_dim] of a PagedKVNeed)."""
        return self.tensors["k"] if self.tensors else None

    @property
    def v(self) -> Optional[torch.Tensor]:
        return self.tensors["v"] if self.tensors else None


@dataclass
class _Group:
    need: PagedNeed
    entries: List[int]
    pool: PagePool
    data: Dict[str, torch.Tensor]    # name -> [n_entries, pages, *leading sizes, page_size, last size]

    def bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.data.values())


def group_needs(needs: Sequence[object], sources: Sequence[Optional[int]]) -> List[PagedNeed]:
    """The page groups that a cache manager makes for these entries, in its order: the distinct
    paged needs in the order in which the entries first ask for them."""
    out: List[PagedNeed] = []
    for need, src in zip(needs, sources):
        if src is None and need is not None:
            paged, _ = needs_of(need)
            if paged is not None and paged not in out:
                out.append(paged)
    return out


class CacheManager:
    def __init__(self, needs: Sequence[object], sources: Sequence[Optional[int]], *,
                 page_size: int, num_pages, max_seqs: int, dtype: torch.dtype,
                 device, page_order_seed: Optional[int] = None):
        """`needs[i]` is what entry i of the execution order needs (None for
        nothing; a PagedNeed, a StateNeed, or a tuple of one paged need and state
        needs), `sources[i]` the entry whose cache it reads instead of its own.
        `num_pages` is the number of pages of every group, or a sequence with one
        number per group (groups are numbered in the order in which the entries
        first ask for them; `group_needs(needs, sources)` lists them)."""
        if page_size <= 0:
            raise ValueError("cache: page_size must be positive")
        self.page_size = int(page_size)
        self.max_seqs = int(max_seqs)
        self.device = torch.device(device)
        self.groups: List[_Group] = []
        self._entry_group: Dict[int, Tuple[int, int]] = {}     # entry -> (group, index in group)
        self._entry_state: Dict[int, Dict[str, torch.Tensor]] = {}
        self._sources = list(sources)
        by_need: Dict[PagedNeed, int] = {}
        for i, need in enumerate(needs):
            if sources[i] is not None or need is None:
                continue
            try:
                paged, states = needs_of(need)
            except (TypeError, ValueError) as e:
                raise type(e)(f"cache: entry {i}: {e}") from None
            if paged is not None:
                names = [t.name for t in paged.tensors]
                if not names or len(set(names)) != len(names) or any(not t.shape or min(t.shape) <= 0 for t in paged.tensors):
                    raise ValueError(f"cache: entry {i} asks for paged tensors {paged.tensors!r}: they need "
                                     f"distinct names and positive sizes")
                if paged not in by_need:
                    by_need[paged] = len(self.groups)
                    self.groups.append(_Group(paged, [], None, None))
                g = by_need[paged]
                self._entry_group[i] = (g, len(self.groups[g].entries))
                self.groups[g].entries.append(i)
            if states:
                self._entry_state[i] = {s.name: torch.zeros((self.max_seqs, *s.shape), dtype=s.dtype, device=self.device)
                                        for s in states}
        ng = len(self.groups)
        if isinstance(num_pages, (int, np.integer)):
            counts = [int(num_pages)] * ng
        else:
            counts = [int(n) for n in num_pages]
            if len(counts) != ng:
                raise ValueError(f"cache: {len(counts)} page counts for {ng} page groups")
        if any(n * self.page_size >= 1 << 31 for n in counts):
            raise ValueError("cache: more than 2^31 token slots in a group")
        orders = None
        if page_order_seed is not None and self.groups:
            orders = []
            for gi in range(ng):
                gen = torch.Generator().manual_seed(page_order_seed + gi)
                orders += torch.randperm(counts[gi], generator=gen).tolist()
        self._lib = native.lib()
        self._book = self._lib.li_book_create(self.page_size, self.max_seqs, ng,
                                              native.int_array([g.need.window for g in self.groups]),
                                              native.int_array(counts), native.int_array(orders) if orders else None)
        err = self._lib.li_book_error(self._book).decode()
        if err:
            self._lib.li_book_destroy(self._book)
            self._book = None
            raise ValueError(err)
        self._ints = (ctypes.c_int * max(ng, 1))()
        for gi, g in enumerate(self.groups):
            g.pool = PagePool(counts[gi], _borrowed=self._lib.li_book_pool(self._book, gi))
            g.data = {t.name: torch.zeros((len(g.entries), counts[gi], *t.page_shape(self.page_size)),
                                          dtype=t.dtype or dtype, device=self.device) for t in g.need.tensors}
        # requests are named by any hashable; the book knows them by number
        self._handles: Dict[Hashable, int] = {}
        self._next_handle = 0

    def __del__(self):
        if getattr(self, "_book", None):
            self._lib.li_book_destroy(self._book)
            self._book = None

    def _error(self) -> str:
        return self._lib.li_book_error(self._book).decode()

    def _handle(self, rid) -> int:
        h = self._handles.get(rid)
        if h is None:
            raise KeyError(rid)
        return h

    # ---- views ---------------------------------------------------------
    def view(self, entry: int) -> CacheView:
        src = self._sources[entry]
        owner = entry if src is None else src
        view = CacheView(owned=src is None)
        if owner in self._entry_group:
            g, j = self._entry_group[owner]
            view.group, view.page_size = g, self.page_size
            view.tensors = {name: d[j] for name, d in self.groups[g].data.items()}
        if owner in self._entry_state:
            view.states = self._entry_state[owner]
            view.state = next(iter(view.states.values()))
        return view

    # ---- requests --------------------------------------------------------
    def has(self, rid) -> bool:
        return rid in self._handles

    def live(self) -> List[Hashable]:
        return list(self._handles)

    def handle(self, rid) -> int:
        """The number under which the host library knows a live request."""
        return self._handle(rid)

    @property
    def book(self):
        return self._book

    def free_slots(self) -> int:
        return self._lib.li_book_free_slots(self._book)

    def free_pages(self) -> List[int]:
        self._lib.li_book_free_pages(self._book, self._ints)
        return list(self._ints[:len(self.groups)])

    def admit(self, rid) -> int:
        if rid in self._handles:
            raise KeyError(f"cache: request {rid!r} is already live")
        h = self._next_handle
        slot = self._lib.li_book_admit(self._book, h)
        if slot == native.ERR_FULL:
            raise CacheFull(self._error())
        if slot < 0:
            raise RuntimeError(self._error())
        self._next_handle += 1
        self._handles[rid] = h
        for states in self._entry_state.values():
            for st in states.values():
                st[slot].zero_()
        return slot

    def slot(self, rid) -> int:
        return self._lib.li_book_slot(self._book, self._handle(rid))

    def cached_len(self, rid) -> int:
        return self._lib.li_book_cached(self._book, self._handle(rid))

    def block_table(self, rid, group: int) -> List[int]:
        h = self._handle(rid)
        n = self._lib.li_book_table_len(self._book, h, group)
        buf = (ctypes.c_int * max(n, 1))()
        self._lib.li_book_table(self._book, h, group, buf, n)
        return list(buf[:n])

    def table_len(self, rid, group: int) -> int:
        return self._lib.li_book_table_len(self._book, self._handle(rid), group)

    def pages_needed(self, rid, n_new: int, cached: Optional[int] = None) -> List[int]:
        """Pages each group must take so that `n_new` more tokens of `rid` fit
        (rid may be unknown: then it is counted as a new request)."""
        h = self._handles.get(rid, -1)
        self._lib.li_book_pages_needed(self._book, h, int(n_new), -1 if cached is None else int(cached), self._ints)
        return list(self._ints[:len(self.groups)])

    # ---- whole batches in one call (the step function and the scheduler go through these) ----
    def handles_of(self, rids, unknown: int = -1) -> "np.ndarray":
        """int64 handles of the requests; `unknown` for one that is not live."""
        get = self._handles.get
        return np.fromiter((get(r, unknown) for r in rids), dtype=np.int64, count=len(rids))

    def pages_needed_many(self, handles, n_new) -> "np.ndarray":
        """[n, groups]: pages each request must take for its n_new[i] more tokens (a handle < 0
        is counted as a new request)."""
        n = len(handles)
        out = np.zeros((n, max(len(self.groups), 1)), dtype=np.int32)
        n_new = np.ascontiguousarray(n_new, dtype=np.int32)
        self._lib.li_book_pages_needed_many(self._book, n, handles.ctypes.data, n_new.ctypes.data, out.ctypes.data)
        return out[:, :len(self.groups)]

    def reserve_many(self, handles, n_new) -> None:
        """Pages for every request of the batch, or none at all (CacheFull)."""
        n_new = np.ascontiguousarray(n_new, dtype=np.int32)
        rc = self._lib.li_book_reserve_many(self._book, len(handles), handles.ctypes.data, n_new.ctypes.data)
        if rc == native.ERR_FULL:
            raise CacheFull(self._error())
        if rc < 0:
            raise PagePoolError(self._error())

    def commit_many(self, handles, n_new) -> None:
        n_new = np.ascontiguousarray(n_new, dtype=np.int32)
        if self._lib.li_book_commit_many(self._book, len(handles), handles.ctypes.data, n_new.ctypes.data) < 0:
            raise PagePoolError(self._error())

    def cached_many(self, handles) -> "np.ndarray":
        """Cached lengths (0 for a handle < 0, a request that is not live yet)."""
        out = np.zeros(len(handles), dtype=np.int32)
        self._lib.li_book_cached_many(self._book, len(handles), handles.ctypes.data, out.ctypes.data)
        return np.maximum(out, 0)

    def max_table_len(self, handles) -> List[int]:
        """The longest block table among the requests, per group."""
        if self._lib.li_book_max_table_len(self._book, len(handles), handles.ctypes.data, self._ints) < 0:
            raise KeyError(self._error())
        return list(self._ints[:len(self.groups)])

    def reserve(self, rid, n_new: int) -> None:
        """Take the pages that positions cached..cached+n_new-1 need, in every
        group, or none at all (CacheFull)."""
        rc = self._lib.li_book_reserve(self._book, self._handle(rid), int(n_new))
        if rc == native.ERR_FULL:
            raise CacheFull(f"{self._error()} (request {rid!r})")
        if rc < 0:
            raise PagePoolError(self._error())

    def commit(self, rid, n_new: int) -> None:
        """`n_new` tokens were written: advance, and give back the pages that
        the window has passed."""
        if self._lib.li_book_commit(self._book, self._handle(rid), int(n_new)) < 0:
            raise PagePoolError(self._error())

    @property
    def has_state(self) -> bool:
        """Whether any mixer keeps per-request state of fixed size in this cache."""
        return bool(self._entry_state)

    def rewind(self, rid, n: int) -> None:
        """Forget the last `n` tokens of `rid`: their positions will be computed and written
        again.  The pages stay with the request.  Refused (ValueError) where a windowed group has
        already given back a page that the earlier position still sees, and where any entry keeps
        state of fixed size: such a state has moved on with the tokens and cannot be taken back."""
        if self._entry_state and n:
            raise ValueError("cache: a request's last tokens cannot be forgotten where a mixer keeps state of fixed "
                             "size (the state has moved on with them)")
        if self._lib.li_book_rewind(self._book, self._handle(rid), int(n)) < 0:
            raise ValueError(self._error())

    def release(self, rid) -> None:
        h = self._handles.pop(rid)
        if self._lib.li_book_release(self._book, h) < 0:
            raise PagePoolError(self._error())

    def check_invariants(self) -> None:
        """No page lost, held twice or on the free list while in a table."""
        if self._lib.li_book_check(self._book) < 0:
            raise AssertionError(self._error())
        if self._lib.li_book_num_live(self._book) != len(self._handles):
            raise AssertionError("the book and the request names disagree")
