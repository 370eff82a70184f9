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
