"""The engine on the GPU against the plain implementation: whole requests,
tails decoded one by one, portions of changing size, mixed batches with pages
used again; in 32-bit and in bfloat16."""
import numpy as np
import pytest
import torch

import helpers
import schedules
from tiny_configs import (TINY_A, TINY_A_PAGE, TINY_B, TINY_B_PAGE, TINY_C, TINY_C_PAGE, TINY_D, TINY_D_PAGE,
                          TINY_E, TINY_E_PAGE)

pytestmark = pytest.mark.gpu

CASES = {"A": (TINY_A, TINY_A_PAGE, 0), "B": (TINY_B, TINY_B_PAGE, 1), "C": (TINY_C, TINY_C_PAGE, 2),
         "D": (TINY_D, TINY_D_PAGE, 3), "E": (TINY_E, TINY_E_PAGE, 4)}
LENGTHS = [5, 17, 33, 70, 100, 41, 64, 2, 1]
# float32: rounding of a different summation order only.  bfloat16: weights are
# bfloat16 on both sides (the plain side computes in float64 from the stored
# values); what differs is the rounding of activations to bfloat16 between kernels.
TOL = {"float32": 2e-5, "bfloat16": 1.5e-2}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, (cfg, page, seed) in CASES.items():
        for dt in ("float32", "bfloat16"):
            stored = torch.float32 if dt == "float32" else torch.bfloat16
            d = helpers.make_model(tmp_path_factory.mktemp(f"m{name}{dt}"), cfg, seed, stored)
            reqs = helpers.random_requests(cfg["vocab_size"], LENGTHS, seed + 10)
            out[(name, dt)] = (d, reqs, helpers.plain_logits(d, reqs))
    return out


def _engine(d, dt, page, max_tokens, **kw):
    from litinfer_amd.engine import Engine
    return Engine.from_dir(d, dtype=dt, device="cuda:0", page_size=page, max_tokens=max_tokens,
                           max_seqs=4, page_order_seed=11, **kw)


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CASES))
@pytest.mark.parametrize("kind", ["whole", "tail", "chunks", "mixed"])
def test_schedules_match_the_plain_implementation(models, name, dt, kind):
    cfg, page, _ = CASES[name]
    d, reqs, ref = models[(name, dt)]
    steps = getattr(schedules, kind)(reqs)
    # the mixed schedule gets exactly the pages its fullest moment needs, so that the pages of a
    # finished request are taken by the next one
    eng = _engine(d, dt, page, schedules.max_live_tokens(reqs, steps, page if kind == "mixed" else 64))
    out = schedules.run(eng, reqs, steps)
    eng.cache.check_invariants()
    assert all(f == g.pool.capacity for f, g in zip(eng.cache.free_pages(), eng.cache.groups))
    if kind == "mixed":
        assert all(g.pool.total_allocations > g.pool.capacity for g in eng.cache.groups), "no page was used again"
    worst = max(schedules.rel_err(out[r], ref[r]) for r in reqs)
    print(f"[observed] {name} {dt} {kind}: {worst:.3e}")
    assert worst < TOL[dt], f"{name} {dt} {kind}: {worst}"


@pytest.mark.parametrize("name", list(CASES))
def test_float32_schedules_agree_with_each_other_closely(models, name):
    cfg, page, _ = CASES[name]
    d, reqs, _ = models[(name, "float32")]
    outs = {}
    for kind in ("whole", "tail", "chunks", "mixed"):
        steps = getattr(schedules, kind)(reqs)
        outs[kind] = schedules.run(_engine(d, "float32", page, schedules.max_live_tokens(reqs, steps)), reqs, steps)
    for kind in ("tail", "chunks", "mixed"):
        for r in reqs:
            assert schedules.rel_err(outs[kind][r], outs["whole"][r].astype(np.float64)) < 5e-6


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_recorded_decode_steps_equal_eager_ones_on_every_replay(models, dt):
    """Decode steps are recorded as HIP graphs and replayed.  Every replay is
    compared with an engine that records nothing, with eager steps (portions of
    another request, a change of the batch's shape) and synchronizations between
    the replays, and across a change of the block table's width."""
    from litinfer_amd.engine import StepEntry
    cfg, page, _ = CASES["B"]
    d, reqs, ref = models[("B", dt)]
    a, b, c = reqs["r4"], reqs["r3"], reqs["r5"]           # 100, 70 and 41 tokens
    engines = [_engine(d, dt, page, 512, use_graphs=g) for g in (True, False)]
    outs = [[], []]
    for eng, out in zip(engines, outs):
        eng.step([StepEntry("a", a[:3], []), StepEntry("b", b[:5], [])])
        for i in range(60):
            batch = [StepEntry("a", [a[3 + i]], [0]), StepEntry("b", [b[5 + i]], [0])]
            out.append(eng.step(batch).clone())
            torch.cuda.synchronize()
            if i % 7 == 3 and (i // 7) * 5 + 5 <= len(c):   # eager work between replays
                lo = (i // 7) * 5
                out.append(eng.step([StepEntry("c", c[lo:lo + 5], [4])]).clone())
                last_c = (len(out) - 1, lo + 4)
            if i == 40:                                    # another shape of batch, once
                out.append(eng.step([StepEntry("a", [a[44]], [0])]).clone())
                out.append(eng.step([StepEntry("b", [b[46]], [0])]).clone())
        out.append(eng.step([StepEntry("a", a[64:70], [5]), StepEntry("b", [b[65]], [0])]).clone())
    assert engines[0].graph_replays >= 50 and engines[1].graph_replays == 0
    assert len(engines[0]._graphs) >= 2                    # the table grew past a width: a second graph
    for x, y in zip(*outs):
        assert torch.equal(x, y)
    # and they are right, not only equal: request c was fed in order between the replays
    at, pos = last_c
    assert schedules.rel_err(outs[0][at].cpu().numpy()[0], ref["r5"][pos]) < TOL[dt]


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "E"])
def test_recorded_steps_filled_up_with_copies_of_the_last_entry(models, name, dt):
    """A recorded decode step of more than four requests is filled up to a multiple of four with copies of its
    last entry, so that one recording serves several numbers of requests.  5 to 11 requests that come and go:
    the logits of every request and step are the plain implementation's, requests that are never last and the
    one that is copied alike, nothing is counted twice in the cache, and few shapes are recorded."""
    from litinfer_amd.engine import StepEntry
    cfg, page, _ = CASES[name]
    d, _, _ = models[(name, dt)]
    lengths = [40, 33, 47, 38, 52, 36, 44, 41, 35, 49, 43]
    reqs = helpers.random_requests(cfg["vocab_size"], lengths, 123)
    ref = helpers.plain_logits(d, reqs)
    from litinfer_amd.engine import Engine
    eng = Engine.from_dir(d, dtype=dt, device="cuda:0", page_size=page, max_tokens=16 * 64, max_seqs=12, graph_after=2)
    assert eng.pad_rows_to == 4
    names = list(reqs)
    at = {}
    for r in names[:5]:                                     # five start with 20 tokens each
        eng.step([StepEntry(r, reqs[r][:20], [])])
        at[r] = 20
    worst, steps = 0.0, 0
    waiting = names[5:]
    while at:
        if waiting and steps % 3 == 2:                      # another request joins, its prompt in one portion
            r = waiting.pop(0)
            eng.step([StepEntry(r, reqs[r][:20], [])])
            at[r] = 20
        live = [r for r in names if r in at]
        out = eng.step([StepEntry(r, [reqs[r][at[r]]], [0]) for r in live])
        assert out.shape[0] == len(live)                    # the copies' rows are not handed out
        got = out.cpu().numpy()
        for i, r in enumerate(live):
            worst = max(worst, schedules.rel_err(got[i], ref[r][at[r]]))
            at[r] += 1
            assert eng.cache.cached_len(r) == at[r]
            if at[r] == len(reqs[r]):
                eng.finish(r)
                del at[r]
        steps += 1
    eng.cache.check_invariants()
    print(f"[observed] {name} {dt}: {worst:.3e}; {eng.graphs_recorded} recordings, {eng.graph_replays} replays in {steps} steps")
    assert worst < TOL[dt]
    assert eng.graph_replays > steps // 2 and eng.graphs_recorded <= 8


@pytest.mark.parametrize("dt,name", [("bfloat16", "D"), ("bfloat16", "E"), ("float32", "B")])
def test_a_long_prompt_in_portions_then_decoding(tmp_path, dt, name):
    """Thousands of positions: many tiles of queries, block tables of hundreds of pages, many
    key splits when decoding; a window far behind the head.  Portions of 2,048 and a ragged
    rest, then tokens one by one, against the plain implementation."""
    from litinfer_amd.engine import StepEntry
    cfg = dict(CASES[name][0], max_position_embeddings=8192)
    page = CASES[name][1]
    stored = torch.float32 if dt == "float32" else torch.bfloat16
    d = helpers.make_model(tmp_path, cfg, 31, stored)
    n, tail = 4500, 6
    toks = helpers.random_requests(cfg["vocab_size"], [n + tail], 32)["r0"]
    ref = helpers.plain_logits(d, {"r0": toks})["r0"]
    eng = _engine(d, dt, page, 4608 + 64)
    got = {}
    start = 0
    for size in (2048, 2048, n - 4096):
        want = [0, size // 2, size - 1]
        out = eng.step([StepEntry("r0", toks[start:start + size], want)]).cpu().numpy()
        for w, row in zip(want, out):
            got[start + w] = row
        start += size
    for i in range(tail):
        got[n + i] = eng.step([StepEntry("r0", [toks[n + i]], [0])]).cpu().numpy()[0]
    worst = max(schedules.rel_err(v, ref[p]) for p, v in got.items())
    print(f"[observed] long prompt {name} {dt}: {worst:.3e}")
    assert worst < TOL[dt], f"{name} {dt}: {worst}"


@pytest.mark.parametrize("stored", [torch.float16, torch.float32])
@pytest.mark.parametrize("name", ["D", "E"])
def test_a_checkpoint_in_another_precision_runs_the_bfloat16_kernels(tmp_path, name, stored):
    """A checkpoint stored in half precision (the reference's own benchmark model is) or in 32-bit,
    in the bfloat16 engine: every matrix is bound as bfloat16, and the mixed schedule matches the
    plain implementation computed from the stored matrices rounded once to bfloat16."""
    cfg, page, seed = CASES[name]
    d = helpers.make_model(tmp_path, cfg, seed + 40, stored)
    reqs = helpers.random_requests(cfg["vocab_size"], LENGTHS, seed + 50)
    ref = helpers.plain_logits(d, reqs, matrices_as_bfloat16=True)
    steps = schedules.mixed(reqs)
    eng = _engine(d, "bfloat16", page, schedules.max_live_tokens(reqs, steps, page))
    layer = eng.model.layers[0]
    assert layer.mixer.qkv.weight.dtype is torch.bfloat16 and layer.ffn.gate_up.weight.dtype is torch.bfloat16
    assert eng.model.head.proj.weight.dtype is torch.bfloat16 and layer.norm1.weight.dtype is torch.float32
    out = schedules.run(eng, reqs, steps)
    worst = max(schedules.rel_err(out[r], ref[r]) for r in reqs)
    print(f"[observed] {name} stored {stored} in the bfloat16 engine, mixed: {worst:.3e}")
    assert worst < TOL["bfloat16"], f"{name} {stored}: {worst}"


def test_a_prompt_of_twelve_thousand_tokens_in_portions_of_2048_then_decoding(tmp_path):
    """The lengths of the long-prompt workload at the engine's level: block tables of hundreds of pages,
    portions of 2,048 behind up to 10,000 cached keys (their keys cut into runs), then single tokens over
    12,000 keys; logits at a few rows of every portion and at every decoded token against the plain
    implementation."""
    from litinfer_amd.engine import StepEntry
    cfg = dict(TINY_E, max_position_embeddings=16384)
    d = helpers.make_model(tmp_path, cfg, 61, torch.bfloat16)
    n, tail = 12000, 8
    toks = helpers.random_requests(cfg["vocab_size"], [n + tail], 62)["r0"]
    ref = helpers.plain_logits(d, {"r0": toks})["r0"]
    eng = _engine(d, "bfloat16", TINY_E_PAGE, n + 64)
    got, start = {}, 0
    while start < n:
        size = min(2048, n - start)
        want = sorted({0, size // 3, size - 1})
        out = eng.step([StepEntry("r0", toks[start:start + size], want)]).cpu().numpy()
        got.update({start + w: row for w, row in zip(want, out)})
        start += size
    for i in range(tail):
        got[n + i] = eng.step([StepEntry("r0", [toks[n + i]], [0])]).cpu().numpy()[0]
    worst = max(schedules.rel_err(v, ref[p]) for p, v in got.items())
    print(f"[observed] prompt of 12,000 tokens in portions of 2,048, then 8 tokens: {worst:.3e}")
    assert worst < TOL["bfloat16"], worst


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "D"])
def test_the_windowed_groups_pool_at_its_minimum(models, name, dt):
    """Every page group has a pool of its own size.  The mixed schedule once with roomy pools, which shows
    the most pages each group ever held at a time, then with exactly that many: the windowed layers' pool
    is a fraction of the other, its pages go round many times, no step runs out, and the logits are the
    plain implementation's."""
    cfg, page, _ = CASES[name]
    d, reqs, ref = models[(name, dt)]
    steps = schedules.mixed(reqs)
    roomy = _engine(d, dt, page, 4 * 128)
    schedules.run(roomy, reqs, steps)
    peaks = [g.pool.peak_used for g in roomy.cache.groups]
    windows = [g.need.window for g in roomy.cache.groups]
    assert windows[0] == 0 and windows[1] == cfg["sliding_window"] and peaks[1] < peaks[0]
    from litinfer_amd.engine import Engine
    eng = Engine.from_dir(d, dtype=dt, device="cuda:0", page_size=page, num_pages=peaks, max_seqs=4, page_order_seed=11)
    assert [g.pool.capacity for g in eng.cache.groups] == peaks
    assert eng.cache.groups[1].data["k"].shape[1] == peaks[1]
    out = schedules.run(eng, reqs, steps)
    eng.cache.check_invariants()
    assert [g.pool.peak_used for g in eng.cache.groups] == peaks and eng.cache.free_pages() == peaks
    assert eng.cache.groups[1].pool.total_allocations > peaks[1]          # its pages were used again
    worst = max(schedules.rel_err(out[r], ref[r]) for r in reqs)
    print(f"[observed] {name} {dt} pools of {peaks} pages: {worst:.3e}")
    assert worst < TOL[dt], worst
