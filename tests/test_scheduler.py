"""The scheduler's decisions, on the CPU with a stand-in engine whose logits
are canned: budget, portions, first come first served, finishing rules,
preemption when pages run out."""
from types import SimpleNamespace

import pytest
import torch

from litinfer_amd.cache import CacheManager
from litinfer_amd.engine import Scheduler
from litinfer_amd.parts import PagedKVNeed
from litinfer_amd.sampling import SamplingParams, uniform

VOCAB = 50


class FakeEngine:
    """Owns a real cache manager; `step` does the bookkeeping of the real one
    and returns logits whose argmax is (last token + 1) % VOCAB."""

    def __init__(self, num_pages=8, page=4, max_seqs=4, max_positions=64, eos=(), windows=(0,)):
        """`windows`: one page group per entry (0: all keys); `num_pages` a number for all or one per group."""
        self.cache = CacheManager([PagedKVNeed(1, 4, w) for w in windows], [None] * len(windows), page_size=page,
                                  num_pages=num_pages, max_seqs=max_seqs, dtype=torch.float32, device="cpu")
        self.spec = SimpleNamespace(vocab_size=VOCAB, max_positions=max_positions, eos_token_ids=tuple(eos))
        self.rt = SimpleNamespace(device=torch.device("cpu"))
        self.batches = []

    def step(self, entries):
        for e in entries:
            if not self.cache.has(e.rid):
                self.cache.admit(e.rid)
        for e in entries:
            self.cache.reserve(e.rid, len(e.tokens))
        rows = []
        for e in entries:
            self.cache.commit(e.rid, len(e.tokens))
            for w in e.want:
                row = torch.zeros(VOCAB)
                row[(e.tokens[w] + 1) % VOCAB] = 5.0
                rows.append(row)
        self.batches.append([(e.rid, len(e.tokens), list(e.want)) for e in entries])
        self.cache.check_invariants()
        return torch.stack(rows) if rows else None

    def finish(self, rid):
        if self.cache.has(rid):
            self.cache.release(rid)


class HostSampler:
    def sample(self, logits, params, counters):
        import torch_ops
        n = logits.shape[0]
        out = torch.empty(n, dtype=torch.int32)
        torch_ops.sample_rows(logits, torch.tensor([p.temperature for p in params]),
                              torch.tensor([p.top_k for p in params]), torch.tensor([p.top_p for p in params]),
                              torch.tensor([uniform(p.seed, c) for p, c in zip(params, counters)]), out)
        return out.tolist()


def sched(engine, **kw):
    return Scheduler(engine, sampler=HostSampler(), **kw)


def test_budget_portions_and_logits_only_at_the_prompts_end():
    e = FakeEngine(num_pages=32)
    s = sched(e, max_batch_tokens=10, chunk_size=6)
    a = s.add_request(list(range(14)), max_new_tokens=3)
    b = s.add_request(list(range(20, 25)), max_new_tokens=2)
    s.run_to_completion()
    assert e.batches[0] == [(a, 6, []), (b, 4, [])]               # budget 10 = 6 + 4, no logits yet
    assert e.batches[1] == [(b, 1, [0]), (a, 6, [])]              # b's prompt ends: one row of logits
    assert e.batches[2] == [(b, 1, [0]), (a, 2, [1])]             # single tokens first, then a's last portion
    assert all(sum(n for _, n, _ in batch) <= 10 for batch in e.batches)
    assert s.output(a) == [14, 15, 16] and s.output(b) == [25, 26]
    assert s.requests[a].finish_reason == "length" and e.cache.free_pages() == [32]


def test_first_come_first_served_and_short_requests_finish_first():
    # the reference's scheduler test: requests of length 2, 5, 10 all finish, in length order
    # (scripts/test_engine_runtime.py:56-83)
    e = FakeEngine(num_pages=32)
    s = sched(e)
    ids = [s.add_request([1, 2, 3], max_new_tokens=n) for n in (10, 2, 5)]
    done = []
    while s.has_unfinished():
        s.step()
        done += [i for i in ids if s.is_finished(i) and i not in done]
    assert done == [ids[1], ids[2], ids[0]]
    assert [r for r, _, _ in e.batches[0]] == ids                  # admitted in arrival order


def test_end_token_is_dropped_and_length_token_is_kept():
    e = FakeEngine(eos=(7,))
    s = sched(e)
    a = s.add_request([4], max_new_tokens=10)                      # 5, 6, then 7 = end: dropped
    b = s.add_request([6], max_new_tokens=10)                      # the very first token is the end token
    c = s.add_request([10], max_new_tokens=2)
    s.run_to_completion()
    assert s.output(a) == [5, 6] and s.requests[a].finish_reason == "eos"
    assert s.output(b) == [] and s.requests[b].finish_reason == "eos"
    assert s.output(c) == [11, 12] and s.requests[c].finish_reason == "length"


def test_submission_checks():
    e = FakeEngine(num_pages=4, page=4, max_positions=32)
    s = sched(e)
    with pytest.raises(ValueError, match="must not be empty"):
        s.add_request([], 4)
    with pytest.raises(ValueError, match="max sequence length"):
        s.add_request(list(range(30)), 4)                          # 30 + 4 - 1 > 32
    with pytest.raises(ValueError, match="could never run"):
        s.add_request(list(range(10)), 10)                         # 19 tokens need 5 pages of 4
    with pytest.raises(ValueError, match="vocabulary"):
        s.add_request([VOCAB], 1)
    s.add_request(list(range(10)), 7)                              # 16 tokens: exactly the pool


def test_out_of_pages_preempts_the_latest_and_tokens_stay_the_same():
    def run(num_pages):
        e = FakeEngine(num_pages=num_pages, page=4, max_seqs=3)
        s = sched(e, max_batch_tokens=64, chunk_size=64)
        ids = [s.add_request([i * 10 + j for j in range(6)], max_new_tokens=9,
                             params=SamplingParams(temperature=0.9, seed=i)) for i in range(3)]
        s.run_to_completion(max_steps=500)
        assert not s.has_unfinished() and e.cache.free_pages() == [num_pages]
        return [s.output(i) for i in ids], s
    plenty, s0 = run(32)
    scarce, s1 = run(8)                     # 3 requests x 15 tokens need 12 pages: they cannot all stay
    assert s0.preemptions == 0 and s1.preemptions > 0
    assert scarce == plenty
    victim = max(s1.requests.values(), key=lambda r: r.preemptions)
    assert victim.rid == 2                  # the most recently admitted one is the one that yields


def test_waiting_request_is_admitted_when_pages_come_back():
    e = FakeEngine(num_pages=4, page=4, max_seqs=4)
    s = sched(e)
    a = s.add_request(list(range(12)), max_new_tokens=4)           # 15 tokens: 4 pages, the whole pool
    b = s.add_request(list(range(5)), max_new_tokens=2)
    s.step()
    assert [r for r, _, _ in e.batches[0]] == [a] and s.requests[b].state == "waiting"
    s.run_to_completion()
    assert s.output(b) == [5, 6] and s.requests[a].preemptions == 0


def test_prompts_cut_into_portions_do_not_share_out_the_pool_and_stall():
    # three prompts of 20 tokens in portions of 4, a pool of 8 pages of 4: each fits alone, two fit
    # together, three do not.  Admitting each on its first portion would leave all three holding
    # pages with none able to finish.
    e = FakeEngine(num_pages=8, page=4, max_seqs=4)
    s = sched(e, max_batch_tokens=12, chunk_size=4)
    ids = [s.add_request([i] * 14, max_new_tokens=3) for i in range(3)]
    s.step()
    assert [r.state for r in s.requests.values()] == ["running", "running", "waiting"]
    s.run_to_completion(max_steps=200)
    assert not s.has_unfinished() and s.preemptions == 0
    assert all(len(s.output(i)) == 3 for i in ids)


def test_a_lone_request_that_outgrows_the_pool_ends_with_an_error():
    e = FakeEngine(num_pages=2, page=4)
    s = sched(e)
    a = s.add_request([1, 2, 3], max_new_tokens=6)
    e.cache.admit("other")                                         # someone else holds a page for good
    e.cache.reserve("other", 4)
    s.run_to_completion(max_steps=50)
    assert s.is_finished(a) and s.requests[a].finish_reason == "error: kv capacity"
    assert len(s.output(a)) == 2                                   # it got as far as its one page allowed


def test_abort_gives_everything_back():
    e = FakeEngine()
    s = sched(e)
    a = s.add_request(list(range(9)), 5)
    s.step()
    s.abort(a)
    assert s.is_finished(a) and e.cache.free_pages() == [8] and not s.has_unfinished()
    assert s.requests[a].finish_reason == "aborted"


def test_sampling_stream_is_per_request():
    # the k-th draw of a request depends on (seed, k) only
    assert uniform(3, 0) == uniform(3, 0) and uniform(3, 0) != uniform(3, 1) != uniform(4, 1)
    assert all(0.0 <= uniform(s, c) < 1.0 for s in range(20) for c in range(50))
    mean = sum(uniform(1, c) for c in range(4000)) / 4000
    assert abs(mean - 0.5) < 0.03


def test_decode_attention_splits_fill_the_simds_in_whole_rounds():
    # every (token, kv head) pair and run of keys is one wave, a SIMD holds one: the runs are chosen for
    # the least rounds x run length, and come four to a block (1, or a multiple of 4)
    from litinfer_amd.kernels.ops import DECODE_MAX_SPLITS, decode_splits
    simds = 1024
    assert decode_splits(8 * 4, 4096, simds) == 32            # 1,024 waves: one round
    assert decode_splits(64 * 4, 4096, simds) == 4
    assert decode_splits(96 * 4, 4096, simds) == 8            # 3 rounds of 512 keys, not 2 of 1,376
    assert decode_splits(24 * 4, 4096, simds) == 8            # 768 waves in one round, not 1,152 in two
    assert decode_splits(24 * 4, 4096, simds, quad=1) == 10   # (single runs: 960 waves)
    assert decode_splits(256 * 4, 4096, simds) == 1
    for pairs in (1, 3, 28, 100, 333, 1000, 5000):
        for keys in (1, 31, 128, 1000, 4096, 100000):
            ns = decode_splits(pairs, keys, simds)
            assert ns == 1 or ns % 4 == 0
            assert 1 <= ns <= DECODE_MAX_SPLITS
            assert ns == 1 or keys / ns >= 96                 # runs of about 128 keys at least


def test_a_step_a_few_tokens_over_whole_tiles_shortens_a_portion():
    # row_tile 8: a portion of 16 beside one decoded token would be 17 tokens, one over two tiles; the
    # portion gives that token up.  A prompt's last portion is never shortened, and nothing is when the
    # step is more than half a tile over.
    e = FakeEngine(num_pages=64, max_positions=200)
    s = sched(e, max_batch_tokens=40, chunk_size=16, row_tile=8)
    a = s.add_request(list(range(3)), max_new_tokens=6)
    s.step()                                                       # a's prompt: 3 tokens, nothing to shorten
    b = s.add_request([(7 * i) % 50 for i in range(50)], max_new_tokens=2)
    s.step()
    assert e.batches[0] == [(a, 3, [2])]
    assert e.batches[1] == [(a, 1, [0]), (b, 15, [])]              # 1 + 16 = 17 -> 16
    s.step()
    assert e.batches[2] == [(a, 1, [0]), (b, 15, [])]
    s.step()
    assert e.batches[3] == [(a, 1, [0]), (b, 15, [])]
    s.step()
    assert e.batches[4] == [(a, 1, [0]), (b, 5, [4])]              # the prompt's end: as it is
    s.run_to_completion()
    assert s.output(a) == [3, 4, 5, 6, 7, 8] and s.output(b) == [44, 45]
    assert e.cache.free_pages() == [64]
    # five tokens over (more than half a tile): as planned
    e2 = FakeEngine(num_pages=64, max_positions=200)
    s2 = sched(e2, max_batch_tokens=40, chunk_size=21, row_tile=8)
    c = s2.add_request([i % 50 for i in range(60)], max_new_tokens=1)
    s2.step()
    assert e2.batches[0] == [(c, 21, [])]
    # and the default leaves every plan alone
    e3 = FakeEngine(num_pages=64, max_positions=200)
    s3 = sched(e3, max_batch_tokens=40, chunk_size=17)
    d = s3.add_request([i % 50 for i in range(60)], max_new_tokens=1)
    s3.step()
    assert e3.batches[0] == [(d, 17, [])]


def test_the_scheduler_takes_the_row_tile_from_the_engine_when_none_is_given():
    e = FakeEngine(num_pages=64, max_positions=200)
    e.row_tile = 8                                                 # what `Engine.row_tile` reports from the model's parts
    s = sched(e, max_batch_tokens=40, chunk_size=16)
    a = s.add_request(list(range(3)), max_new_tokens=6)
    s.step()
    b = s.add_request([(7 * i) % 50 for i in range(50)], max_new_tokens=2)
    s.step()
    assert s.row_tile == 8 and e.batches[1] == [(a, 1, [0]), (b, 15, [])]
    assert sched(FakeEngine(), row_tile=1).row_tile == 1 and sched(FakeEngine()).row_tile == 1


def test_a_small_pool_of_a_windowed_group_admits_long_prompts():
    """The windowed group's pool (6 pages) is smaller than the pages a 40-token prompt fills (10): the
    request is admitted all the same, because at a time it holds the window's pages and a portion's."""
    e = FakeEngine(num_pages=[32, 6], windows=(0, 6), max_positions=200)
    s = sched(e, max_batch_tokens=8, chunk_size=8)
    a = s.add_request([i % 50 for i in range(40)], max_new_tokens=5)
    s.run_to_completion()
    assert s.requests[a].finish_reason == "length" and s.output(a) == [40, 41, 42, 43, 44]
    assert s.preemptions == 0 and e.cache.free_pages() == [32, 6]
    assert e.cache.groups[1].pool.total_allocations >= 11          # its pages went round
    # a portion larger than the windowed pool can hold is cut to what fits
    e2 = FakeEngine(num_pages=[32, 3], windows=(0, 6), max_positions=200)
    s2 = sched(e2, max_batch_tokens=16, chunk_size=16)
    with pytest.raises(ValueError, match="could never run"):
        sched(FakeEngine(num_pages=[32, 2], windows=(0, 6), max_positions=200)).add_request([1] * 9, 2)
    b = s2.add_request([i % 50 for i in range(30)], max_new_tokens=2)
    s2.run_to_completion()
    assert s2.output(b) == [30, 31] and max(n for batch in e2.batches for _, n, _ in batch) <= 12
    assert e2.cache.free_pages() == [32, 3]


def test_unequal_pools_admission_waits_and_preemption_frees_the_windowed_group():
    """Two page groups of unequal pools.  A request is admitted only when BOTH groups have room for what
    it holds at a time; when the windowed group runs out among decoding requests, the last admitted
    gives way and is computed again; tokens are as without the squeeze."""
    prompts = [[(3 * i + k) % 50 for i in range(n)] for k, n in enumerate((14, 9, 11))]

    def run(pages):
        e = FakeEngine(num_pages=pages, windows=(0, 8), max_positions=200, max_seqs=3)
        s = sched(e, max_batch_tokens=12, chunk_size=4)
        ids = [s.add_request(p, max_new_tokens=12) for p in prompts]
        steps = 0
        while s.has_unfinished():
            s.step()
            steps += 1
            assert steps < 400
            e.cache.check_invariants()
        assert e.cache.free_pages() == list(pages)
        return e, s, [s.output(i) for i in ids]
    roomy_e, roomy_s, want = run([64, 64])
    assert roomy_s.preemptions == 0 and all(len(t) == 12 for t in want)
    # window 8, page 4, portions of 4: a request holds up to ceil(11 / 4) + 1 = 4 pages at a time; seven pages
    # do not hold three requests, so the third waits although the full group has room for all
    e, s, got = run([64, 7])
    assert got == want
    first_batches = [sorted(r for r, _, _ in b) for b in e.batches[:3]]
    assert all(len(b) <= 2 for b in first_batches), first_batches
    # a full group too small for all three: the same through the other pool
    e, s, got = run([12, 64])
    assert got == want and (s.preemptions > 0 or any(len(b) < 3 for b in e.batches))
    # both tight: preemption happens and nothing is lost
    e, s, got = run([9, 5])
    assert got == want
