"""The cache manager: no page lost, held twice or freed twice, under random
orders of requests; windows give pages back; state slots."""
import random

import pytest
import torch

from litinfer_amd.cache import CacheFull, CacheManager, PagePool, PagePoolError
from litinfer_amd.parts import PagedKVNeed, PagedNeed, PagedTensor, StateNeed


def test_pool_guards():
    p = PagePool(3)
    a, b, c = p.alloc(), p.alloc(), p.alloc()
    assert sorted((a, b, c)) == [0, 1, 2] and p.free == 0 and a == 0      # the first alloc gives page 0
    with pytest.raises(PagePoolError, match="no free page"):
        p.alloc()
    p.release(b)
    with pytest.raises(PagePoolError, match="freed twice"):
        p.release(b)
    with pytest.raises(PagePoolError, match="out of range"):
        p.release(7)
    assert p.alloc() == b and p.used == 3
    assert PagePool(4, order=[2, 0, 3, 1]).alloc() == 2
    with pytest.raises(ValueError):
        PagePool(3, order=[0, 0, 1])


def _manager(num_pages=12, page=4, window=0, max_seqs=3, seed=None):
    needs = [PagedKVNeed(2, 8, 0), PagedKVNeed(2, 8, window), PagedKVNeed(2, 8, window), None]
    return CacheManager(needs, [None, None, None, None], page_size=page, num_pages=num_pages,
                        max_seqs=max_seqs, dtype=torch.float32, device="cpu", page_order_seed=seed)


def test_groups_by_need_and_views():
    m = _manager(window=6)
    assert len(m.groups) == 2 and m.groups[0].entries == [0] and m.groups[1].entries == [1, 2]
    assert set(m.groups[1].data) == {"k", "v"} and m.groups[1].data["k"].shape == (2, 12, 2, 4, 8)
    v = m.view(2)
    assert v.owned and v.group == 1 and v.k.shape == (12, 2, 4, 8)
    assert v.k.data_ptr() == m.groups[1].data["k"][1].data_ptr()
    assert m.view(3).group is None
    one = _manager(window=0)
    assert len(one.groups) == 1 and one.groups[0].entries == [0, 1, 2]


def test_pages_of_any_named_tensors_group_by_their_need():
    """A need is a list of named tensors per token: keys alone, a latent of another dtype
    beside a small vector, keys and values of unequal head sizes."""
    latent = PagedNeed((PagedTensor("c", (24,), torch.float32), PagedTensor("pe", (2, 6))), window=0)
    uneven = PagedNeed((PagedTensor("k", (2, 16)), PagedTensor("v", (2, 8))), window=5)
    needs = [latent, PagedKVNeed(2, 8, 0), uneven, latent, PagedKVNeed(2, 8, 0)]
    m = CacheManager(needs, [None] * 5, page_size=4, num_pages=6, max_seqs=2, dtype=torch.bfloat16, device="cpu")
    assert [g.entries for g in m.groups] == [[0, 3], [1, 4], [2]]
    assert m.groups[0].data["c"].shape == (2, 6, 4, 24) and m.groups[0].data["c"].dtype is torch.float32
    assert m.groups[0].data["pe"].shape == (2, 6, 2, 4, 6) and m.groups[0].data["pe"].dtype is torch.bfloat16
    assert m.groups[2].data["k"].shape == (1, 6, 2, 4, 16) and m.groups[2].data["v"].shape == (1, 6, 2, 4, 8)
    v = m.view(3)
    assert set(v.tensors) == {"c", "pe"} and v.tensors["c"].shape == (6, 4, 24)
    assert latent.bytes_per_token(torch.bfloat16) == 24 * 4 + 12 * 2
    m.admit("a")
    m.reserve("a", 9)
    m.commit("a", 9)
    assert m.free_pages() == [3, 3, 4]                 # the windowed group has given its first page back
    m.check_invariants()
    with pytest.raises(ValueError, match="distinct names"):
        CacheManager([PagedNeed((PagedTensor("k", (2,)), PagedTensor("k", (2,))))], [None], page_size=4,
                     num_pages=2, max_seqs=1, dtype=torch.float32, device="cpu")
    with pytest.raises(TypeError):
        CacheManager(["pages please"], [None], page_size=4, num_pages=2, max_seqs=1, dtype=torch.float32, device="cpu")


def test_shared_cache_view_is_the_owners():
    m = CacheManager([PagedKVNeed(1, 4, 0), PagedKVNeed(1, 4, 0)], [None, 0], page_size=4, num_pages=2,
                     max_seqs=1, dtype=torch.float32, device="cpu")
    assert m.groups[0].entries == [0]                 # the reader owns no cache
    assert m.view(1).k.data_ptr() == m.view(0).k.data_ptr() and not m.view(1).owned and m.view(0).owned


def test_reserve_is_all_or_nothing_and_commit_advances():
    m = _manager(num_pages=5, page=4)
    m.admit("a")
    m.reserve("a", 9)                                  # 3 pages
    m.commit("a", 9)
    assert m.cached_len("a") == 9 and m.free_pages() == [2]
    m.admit("b")
    with pytest.raises(CacheFull):
        m.reserve("b", 9)
    assert m.free_pages() == [2] and m.block_table("b", 0) == []
    m.reserve("a", 3)                                  # fills page 3 exactly: no new page
    assert m.free_pages() == [2]
    m.release("a")
    m.release("b")
    assert m.free_pages() == [5]
    m.check_invariants()


def test_window_gives_pages_back_and_never_the_visible_ones():
    m = _manager(num_pages=12, page=4, window=6)
    m.admit("a")
    total = 0
    seen_pages = []
    for n in (5, 3, 1, 1, 7, 2, 1, 1, 1, 6, 1, 1, 9, 1, 4):
        m.reserve("a", n)
        m.commit("a", n)
        total += n
        table = m.block_table("a", 1)
        first_visible = max(0, total - 6 + 1)          # what the NEXT query (at `total`) can see
        for b, page in enumerate(table):
            last_pos = (b + 1) * 4 - 1
            if last_pos >= first_visible:
                assert page >= 0, "a page that a later query can see was given back"
            else:
                assert page == -1, "a page that the window has passed is still held"
        assert all(p >= 0 for p in m.block_table("a", 0))      # the full group keeps everything
        assert m.groups[1].pool.used <= 3                      # 6 positions span at most 3 pages of 4
        seen_pages += [p for p in table if p >= 0]
        m.check_invariants()
    assert total == 44 and m.groups[0].pool.used == 11
    assert m.groups[1].pool.total_allocations == 11 and len(set(seen_pages)) < 11   # pages were used again
    m.release("a")
    assert m.free_pages() == [12, 12]


def test_rewind_forgets_tokens_keeps_pages_and_respects_the_window():
    m = _manager(num_pages=6, page=4)
    m.admit("a")
    m.reserve("a", 9)
    m.commit("a", 9)
    table = m.block_table("a", 0)
    m.rewind("a", 2)
    assert m.cached_len("a") == 7 and m.block_table("a", 0) == table and m.free_pages() == [3]
    m.reserve("a", 2)                                  # the same places again: no new page
    m.commit("a", 2)
    assert m.cached_len("a") == 9 and m.block_table("a", 0) == table
    with pytest.raises(ValueError):
        m.rewind("a", 10)
    m.check_invariants()
    w = _manager(num_pages=12, page=4, window=6)
    w.admit("a")
    w.reserve("a", 20)
    w.commit("a", 20)                                  # the windowed group has given back blocks 0..2
    w.rewind("a", 1)                                   # position 19 sees keys from 14 on: block 3, still held
    with pytest.raises(ValueError, match="given back"):
        w.rewind("a", 4)                               # position 15 would see key 10 in block 2, which is gone
    assert w.cached_len("a") == 19
    w.check_invariants()


def test_slots_and_state_are_zeroed_at_admission():
    m = CacheManager([StateNeed((3,), torch.float32), PagedKVNeed(1, 4, 0)], [None, None], page_size=4,
                     num_pages=4, max_seqs=2, dtype=torch.float32, device="cpu")
    s = m.admit("a")
    m.view(0).state[s] += 5
    m.admit("b")
    with pytest.raises(CacheFull, match="state slots"):
        m.admit("c")
    with pytest.raises(KeyError):
        m.admit("a")
    m.release("a")
    s2 = m.admit("c")
    assert s2 == s and torch.equal(m.view(0).state[s2], torch.zeros(3))
    m.check_invariants()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_lose_no_page(seed):
    rng = random.Random(seed)
    m = _manager(num_pages=10, page=4, window=rng.choice([0, 5, 9]), max_seqs=3, seed=seed)
    live, n_done, next_id = {}, 0, 0
    for _ in range(400):
        act = rng.random()
        if act < 0.25 and len(live) < 3:
            rid = f"r{next_id}"
            next_id += 1
            m.admit(rid)
            live[rid] = 0
        elif act < 0.85 and live:
            rid = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 3, 7, 13])
            before = (m.free_pages(), [list(m.block_table(rid, g)) for g in range(len(m.groups))])
            try:
                m.reserve(rid, n)
            except CacheFull:
                assert (m.free_pages(), [list(m.block_table(rid, g)) for g in range(len(m.groups))]) == before
            else:
                m.commit(rid, n)
                live[rid] += n
                assert m.cached_len(rid) == live[rid]
        elif live:
            rid = rng.choice(list(live))
            m.release(rid)
            del live[rid]
            n_done += 1
        m.check_invariants()
        for g in m.groups:
            assert g.pool.used + g.pool.free == g.pool.capacity
    for rid in list(live):
        m.release(rid)
    assert m.free_pages() == [10] * len(m.groups) and m.free_slots() == 3
    with pytest.raises(KeyError):
        m.release("r0")                                 # a request cannot be released twice


def test_an_entry_may_keep_pages_and_states_of_fixed_size_together():
    """One paged need and any number of named states for one entry: its view has both."""
    both = (PagedKVNeed(1, 4, 0), StateNeed((3, 2), torch.float32, name="tail"), StateNeed((5,), torch.int32, name="count"))
    m = CacheManager([both, PagedKVNeed(1, 4, 0), StateNeed((2,))], [None, None, None], page_size=4, num_pages=5,
                     max_seqs=2, dtype=torch.float32, device="cpu")
    assert len(m.groups) == 1 and m.groups[0].entries == [0, 1]          # the paged part joins its group as ever
    v = m.view(0)
    assert v.k.shape == (5, 1, 4, 4) and set(v.states) == {"tail", "count"}
    assert v.state is v.states["tail"] and v.states["tail"].shape == (2, 3, 2) and v.states["count"].dtype is torch.int32
    assert m.view(1).states is None and m.view(1).k is not None
    assert m.view(2).tensors is None and m.view(2).state.shape == (2, 2)
    s = m.admit("a")
    v.states["tail"][s] += 1
    v.states["count"][s] += 7
    m.release("a")
    assert m.admit("b") == s and not v.states["tail"][s].any() and not v.states["count"][s].any()
    m.reserve("b", 3)
    m.commit("b", 3)
    with pytest.raises(ValueError, match="state of fixed size"):
        m.rewind("b", 1)                                                   # the states have moved on with the tokens
    with pytest.raises(ValueError, match="ONE paged need"):
        CacheManager([(PagedKVNeed(1, 4, 0), PagedKVNeed(1, 4, 3))], [None], page_size=4, num_pages=5, max_seqs=2,
                     dtype=torch.float32, device="cpu")
    with pytest.raises(ValueError, match="distinct names"):
        CacheManager([(StateNeed((1,)), StateNeed((2,)))], [None], page_size=4, num_pages=5, max_seqs=2,
                     dtype=torch.float32, device="cpu")
    with pytest.raises(TypeError, match="neither"):
        CacheManager([("pages",)], [None], page_size=4, num_pages=5, max_seqs=2, dtype=torch.float32, device="cpu")


def test_every_group_has_a_pool_of_its_own_size():
    from litinfer_amd.cache import group_needs
    needs = [PagedKVNeed(2, 8, 0), PagedKVNeed(2, 8, 6), PagedKVNeed(2, 8, 6), None]
    assert [n.window for n in group_needs(needs, [None] * 4)] == [0, 6]
    m = CacheManager(needs, [None] * 4, page_size=4, num_pages=[12, 4], max_seqs=2, dtype=torch.float32, device="cpu",
                     page_order_seed=3)
    assert [g.pool.capacity for g in m.groups] == [12, 4] and m.free_pages() == [12, 4]
    assert m.groups[0].data["k"].shape[1] == 12 and m.groups[1].data["k"].shape == (2, 4, 2, 4, 8)
    m.admit("a")
    with pytest.raises(CacheFull, match="of 4 are free"):
        m.reserve("a", 17)                           # five pages at once: the full group could, the windowed cannot
    assert m.free_pages() == [12, 4]
    for _ in range(10):                              # 40 tokens, four at a time: the window's pages go round
        m.reserve("a", 4)
        m.commit("a", 4)
        m.check_invariants()
    assert m.free_pages() == [2, 2] and m.groups[1].pool.total_allocations == 10
    assert all(0 <= p < 4 for p in m.block_table("a", 1) if p >= 0)
    m.release("a")
    assert m.free_pages() == [12, 4]
    with pytest.raises(ValueError, match="page counts"):
        CacheManager(needs, [None] * 4, page_size=4, num_pages=[12], max_seqs=2, dtype=torch.float32, device="cpu")
