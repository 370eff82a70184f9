"""The four schedules on the CPU with the torch stand-ins: they check the
batch layout, the block tables, the page reuse and the window's give-back
where there is no GPU.  The GPU twin is tests/test_engine_gpu.py."""
import pytest

import helpers
import schedules
from litinfer_amd.engine import Engine
from tiny_configs import TINY_A, TINY_A_PAGE, TINY_B, TINY_B_PAGE


@pytest.mark.parametrize("cfg,page,seed", [(TINY_A, TINY_A_PAGE, 0), (TINY_B, TINY_B_PAGE, 1)])
def test_schedules_on_the_stand_ins(tmp_path, cpu_ops, cfg, page, seed):
    d = helpers.make_model(tmp_path, cfg, seed)
    reqs = helpers.random_requests(cfg["vocab_size"], [5, 17, 33, 70, 41, 2, 1], seed + 10)
    ref = helpers.plain_logits(d, reqs)
    for kind in ("whole", "tail", "chunks", "mixed"):
        steps = getattr(schedules, kind)(reqs)
        eng = Engine.from_dir(d, dtype="float32", device="cpu", page_size=page, max_seqs=4, page_order_seed=2,
                              max_tokens=schedules.max_live_tokens(reqs, steps, page if kind == "mixed" else 64))
        out = schedules.run(eng, reqs, steps)
        eng.cache.check_invariants()
        assert all(f == g.pool.capacity for f, g in zip(eng.cache.free_pages(), eng.cache.groups))
        if kind == "mixed":
            assert all(g.pool.total_allocations > g.pool.capacity for g in eng.cache.groups)
        assert max(schedules.rel_err(out[r], ref[r]) for r in reqs) < 2e-5, kind


def test_no_gpu_means_an_error_not_a_fallback(tmp_path):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is visible")
    d = helpers.make_model(tmp_path, TINY_A, 0)
    with pytest.raises(RuntimeError, match="no CPU path"):
        Engine.from_dir(d, dtype="float32", device="cuda:0", max_tokens=64)
    from litinfer_amd.kernels import ops
    with pytest.raises(RuntimeError, match="not on the GPU"):
        ops.rmsnorm(torch.zeros(2, 4), torch.ones(4), 1e-6, torch.zeros(2, 4))


def test_a_forward_that_raises_leaves_no_request_behind(tmp_path, cpu_ops, monkeypatch):
    from litinfer_amd.engine import StepEntry
    d = helpers.make_model(tmp_path, TINY_A, 0)
    eng = Engine.from_dir(d, dtype="float32", device="cpu", page_size=16, max_seqs=2, max_tokens=128)
    eng.step([StepEntry("old", [1, 2, 3], [])])
    free = eng.cache.free_pages()
    real = eng.model.forward

    def broken(ctx, cache):
        raise ValueError("a kernel refused the size")
    monkeypatch.setattr(eng.model, "forward", broken)
    with pytest.raises(ValueError, match="refused"):
        eng.step([StepEntry("old", [4] * 20, []), StepEntry("new", [5, 6], [1])])
    assert not eng.cache.has("new") and eng.cache.cached_len("old") == 3
    assert eng.cache.free_slots() == 1
    eng.cache.check_invariants()
    monkeypatch.setattr(eng.model, "forward", real)
    # the request that was live goes on as if nothing had happened; its reserved pages are used now
    ref = helpers.plain_logits(d, {"r": [1, 2, 3] + [4] * 20})["r"]
    got = eng.step([StepEntry("old", [4] * 20, [19])]).numpy()
    assert schedules.rel_err(got[0], ref[22]) < 2e-5
    eng.finish("old")
    assert eng.cache.free_pages() == [f + 1 for f in free]


class _AddressGraph:
    """Stands in for a recorded graph on the CPU: at the end of recording it remembers where every
    workspace buffer and the batch's device buffer lay, a replay fails if one of them has moved
    since (on the GPU it would write through a stale address), and otherwise runs the forward pass
    that was recorded."""
    engine = None
    stale_replays = 0

    def __init__(self):
        self.addresses = self.call = None

    def replay(self):
        eng = _AddressGraph.engine
        now = {k: b.data_ptr() for k, b in eng.ws._bufs.items()}
        now["batch"] = eng._uploader._dev.data_ptr()
        if any(now.get(k) != p for k, p in self.addresses.items()):
            _AddressGraph.stale_replays += 1
        out = self.call()
        if self.out is not None:                     # (a step that wants no logits has none)
            self.out.copy_(out)


def _graphs_on_the_cpu(eng, monkeypatch):
    """Recording and replaying, with `_AddressGraph` for the GPU's graphs."""
    import contextlib
    import torch
    _AddressGraph.engine, _AddressGraph.stale_replays = eng, 0
    eng.use_graphs = True
    real_forward = eng.model.forward

    @contextlib.contextmanager
    def recording(graph):
        calls = []

        def forward(ctx, cache):
            out = real_forward(ctx, cache)
            graph.out = out
            # what a replay runs: the same forward over the same (re-filled) device arrays
            calls.append(lambda: real_forward(eng._last_ctx, cache))
            return out
        monkeypatch.setattr(eng.model, "forward", forward)
        try:
            yield
        finally:
            monkeypatch.setattr(eng.model, "forward", real_forward)
        graph.call = calls[0]
        graph.addresses = {k: b.data_ptr() for k, b in eng.ws._bufs.items()}
        graph.addresses["batch"] = eng._uploader._dev.data_ptr()
    def record(ctx):                                 # in the place of Engine._record, which records on a stream of the GPU
        graph = _AddressGraph()
        with recording(graph):
            out = eng.model.forward(ctx, eng.cache)
        return graph, out
    monkeypatch.setattr(eng, "_record", record)
    monkeypatch.setattr(torch.cuda, "synchronize", lambda *a, **k: None)
    real_build = eng._build_context

    def build(entries, **kw):
        eng._last_ctx = real_build(entries, **kw)
        return eng._last_ctx
    monkeypatch.setattr(eng, "_build_context", build)


def test_a_buffer_that_grows_between_replays_drops_what_was_recorded(tmp_path, cpu_ops, monkeypatch):
    """A decode batch of 2 is recorded and replayed; then a first decode batch of 9 makes workspace
    buffers grow during its own eager pass; when the batch is 2 again its old recording addresses
    buffers that have moved and must not be replayed: it is recorded anew, and the logits stay right."""
    from litinfer_amd.engine import StepEntry
    d = helpers.make_model(tmp_path, TINY_A, 0)
    eng = Engine.from_dir(d, dtype="float32", device="cpu", page_size=16, max_seqs=12, max_tokens=12 * 64,
                          graph_after=2)
    _graphs_on_the_cpu(eng, monkeypatch)
    reqs = helpers.random_requests(256, [40] * 9, 3)
    ref = helpers.plain_logits(d, reqs)
    at = {r: 1 for r in reqs}
    for r in reqs:                                   # one token each, one by one: no buffer larger than a decode step's
        eng.step([StepEntry(r, reqs[r][:1], [])])
    eng.graph_replays = eng.graphs_recorded = 0      # (those steps were of one shape too)

    def decode(names):
        out = eng.step([StepEntry(r, [reqs[r][at[r]]], [0]) for r in names]).numpy().copy()
        for i, r in enumerate(names):
            assert schedules.rel_err(out[i], ref[r][at[r]]) < 2e-5, (r, at[r])
            at[r] += 1
    two, nine = ["r0", "r1"], list(reqs)
    for _ in range(5):
        decode(two)
    assert eng.graph_replays == 3 and eng.graphs_recorded == 1
    before = eng.ws.generation
    decode(nine)                                     # first of its shape: eager, and larger than anything before
    assert eng.ws.generation > before, "the test needs a buffer to move here"
    for _ in range(4):
        decode(two)                                  # eager + recorded again, then replayed
    assert _AddressGraph.stale_replays == 0, "a recording was replayed after a buffer it addresses had moved"
    assert eng.graphs_recorded == 2 and eng.graph_replays == 6
    for _ in range(3):
        decode(nine)
    assert _AddressGraph.stale_replays == 0 and eng.graphs_recorded == 3


def test_recorded_shapes_are_kept_up_to_a_number_and_recorded_again_after_they_went(tmp_path, cpu_ops, monkeypatch):
    from litinfer_amd.engine import StepEntry
    d = helpers.make_model(tmp_path, TINY_A, 0)
    eng = Engine.from_dir(d, dtype="float32", device="cpu", page_size=16, max_seqs=6, max_tokens=6 * 128,
                          graph_after=2, max_graphs=2)
    _graphs_on_the_cpu(eng, monkeypatch)
    reqs = helpers.random_requests(256, [100] * 5, 4)
    ref = helpers.plain_logits(d, reqs)
    eng.step([StepEntry(r, reqs[r][:2], []) for r in reqs])          # the largest batch first: buffers are sized
    at = {r: 2 for r in reqs}

    def decode(n):
        names = list(reqs)[:n]
        out = eng.step([StepEntry(r, [reqs[r][at[r]]], [0]) for r in names]).numpy().copy()
        for i, r in enumerate(names):
            assert schedules.rel_err(out[i], ref[r][at[r]]) < 2e-5
            at[r] += 1
    decode(5)                                        # the largest decode batch once: its buffers are sized too
    for n in (1, 2, 3, 4):
        for _ in range(3):
            decode(n)
    recorded = [k for k, s in eng._graphs.items() if s[0] == "graph"]
    assert eng.graphs_recorded == 4 and [k[0] for k in recorded] == [3, 4]      # the two used last
    replays = eng.graph_replays
    for _ in range(3):
        decode(1)                                    # went: seen anew, recorded at its second step, replayed at the third
    assert eng.graphs_recorded == 5 and eng.graph_replays == replays + 1
    assert [k[0] for k, s in eng._graphs.items() if s[0] == "graph"] == [4, 1]
    assert _AddressGraph.stale_replays == 0
