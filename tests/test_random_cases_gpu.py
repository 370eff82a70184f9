"""Many small random cases, fixed seeds: mixed schedules of every tiny configuration with random request
lengths, portions, page sizes and numbers of live requests against the plain implementation, and random
decode batches (contexts around the edges of blocks of keys and of pages, windows, head layouts, equal and
unequal contexts, with and without a workspace) of the attention op against the plain attention."""
import numpy as np
import pytest
import torch

import helpers
import schedules
import test_kernels_gpu as kernel_cases
from tiny_configs import (TINY_A, TINY_A_PAGE, TINY_B, TINY_B_PAGE, TINY_C, TINY_C_PAGE, TINY_D, TINY_D_PAGE,
                          TINY_E, TINY_E_PAGE)

pytestmark = pytest.mark.gpu

CASES = {"A": (TINY_A, TINY_A_PAGE, 0), "B": (TINY_B, TINY_B_PAGE, 1), "C": (TINY_C, TINY_C_PAGE, 2),
         "D": (TINY_D, TINY_D_PAGE, 3), "E": (TINY_E, TINY_E_PAGE, 4)}
TOL = {"float32": 2e-5, "bfloat16": 1.5e-2}


@pytest.fixture(scope="module")
def ops():
    from litinfer_amd.kernels import ops
    ops.require_gpu("cuda:0")
    return ops


LENGTHS = [1, 2, 3, 15, 16, 17, 31, 32, 33, 47, 63, 64, 65, 90, 127, 128, 129, 200, 260]
PORTIONS = [2, 3, 5, 8, 16, 17, 31, 32, 33, 64, 100]


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CASES))
def test_random_mixed_schedules_match_the_plain_implementation(tmp_path, name, dt):
    from litinfer_amd.engine import Engine
    cfg, page0, seed = CASES[name]
    d = helpers.make_model(tmp_path, cfg, seed, torch.float32 if dt == "float32" else torch.bfloat16)
    worst = 0.0
    for trial in range(5):
        rng = np.random.default_rng(1000 * trial + seed)
        lengths = [min(int(x), int(cfg["max_position_embeddings"])) for x in rng.choice(LENGTHS, int(rng.integers(3, 9)))]
        reqs = helpers.random_requests(cfg["vocab_size"], lengths, 77 + trial)
        ref = helpers.plain_logits(d, reqs)
        portions = tuple(int(x) for x in rng.choice(PORTIONS, 5))
        page = int(rng.choice([page0, 1, 4, 16, 32])) if trial % 2 else page0
        steps = schedules.mixed(reqs, max_live=int(rng.integers(1, 5)), seed=trial, prefill_chunks=portions,
                                decode_after=float(rng.choice([0.2, 0.6, 0.9])))
        eng = Engine.from_dir(d, dtype=dt, device="cuda:0", page_size=page, max_seqs=4, page_order_seed=trial,
                              max_tokens=schedules.max_live_tokens(reqs, steps, page))
        out = schedules.run(eng, reqs, steps)
        eng.cache.check_invariants()
        assert all(f == g.pool.capacity for f, g in zip(eng.cache.free_pages(), eng.cache.groups))
        err = max(schedules.rel_err(out[r], ref[r]) for r in reqs)
        assert err < TOL[dt], f"{name} {dt} trial {trial}: lengths {lengths}, portions {portions}, page {page}: {err}"
        worst = max(worst, err)
    print(f"[observed] {name} {dt}: {worst:.3e}")


EDGES = [1, 2, 31, 32, 33, 63, 64, 65, 95, 96, 97, 127, 128, 129, 255, 256, 257, 511, 513, 1023, 1024, 1025, 2047,
         2049, 3000, 4095, 4097, 6000]
LAYOUTS = [(28, 4, 128), (12, 2, 128), (40, 8, 128), (14, 2, 64), (7, 7, 128), (40, 2, 64), (16, 1, 128)]


@pytest.mark.parametrize("block", range(4))
def test_random_decode_batches_match_the_plain_attention(ops, block):
    from litinfer_amd.engine.workspace import Workspace
    ws = Workspace("cuda:0")
    rng = np.random.default_rng(5 + block)
    for trial in range(30):
        nh, nkv, dh = LAYOUTS[int(rng.integers(len(LAYOUTS)))]
        page = int(rng.choice([1, 3, 5, 8, 12, 16, 16, 16, 24, 48, 64]))
        window = int(rng.choice([0, 0, 0, 40, 300, 1000]))
        nreq = int(rng.choice([1, 2, 3, 8, 17, 40]))
        longest = 1500 if page == 1 else 10 ** 9
        first = min(int(rng.choice(EDGES)), longest)
        equal = rng.random() < 0.4
        segs = [(first if equal else min(int(rng.choice(EDGES)), longest), 1) for _ in range(nreq)]
        if rng.random() < 0.2:                         # a portion of a prompt beside the decoding requests
            a, b = int(rng.choice([70, 300, 700])), int(rng.choice([2, 33, 70]))
            segs.append((max(a, b), min(a, b)))
        dtype = torch.bfloat16 if rng.random() < 0.6 else torch.float32
        pad = bool(rng.random() < 0.3) and all(q == 1 for _, q in segs)
        out, ref = kernel_cases._paged_case(ops, dtype, segs, nh, nkv, dh, page, window, seed=100 * block + trial,
                                            ws=ws if rng.random() < 0.8 else None, pad_pow2=pad)
        err = kernel_cases.rel(out, ref)
        assert err < kernel_cases.tol(dtype, 3e-6, 1.5e-2), (
            f"block {block} trial {trial}: {dtype} heads {nh}/{nkv}/{dh} page {page} window {window} widened {pad} "
            f"(context, tokens) {segs}: {err}")


PROMPT_LAYOUTS = [(28, 4, 128), (12, 2, 128), (40, 8, 128), (14, 2, 64), (7, 7, 128), (20, 2, 64), (6, 1, 128), (9, 1, 64)]


@pytest.mark.parametrize("block", range(2))
def test_random_prompt_portions_match_the_plain_attention(ops, block):
    """Portions of 2 to 400 queries behind 0 to 4,000 cached keys, one to five requests a call, now and then a
    decoding request beside them."""
    from litinfer_amd.engine.workspace import Workspace
    ws = Workspace("cuda:0")
    rng = np.random.default_rng(11 + block)
    for trial in range(40):
        nh, nkv, dh = PROMPT_LAYOUTS[int(rng.integers(len(PROMPT_LAYOUTS)))]
        page = int(rng.choice([1, 3, 5, 8, 12, 16, 16, 16, 24, 48, 64]))
        window = int(rng.choice([0, 0, 0, 40, 300, 1000]))
        segs = []
        for _ in range(int(rng.choice([1, 1, 2, 3, 5]))):
            q = int(rng.choice([2, 3, 31, 32, 33, 64, 65, 100, 257, 400]))
            before = int(rng.choice([0, 0, 1, 31, 32, 33, 500, 1500, 4000]))
            segs.append(((min(before, 700) if page == 1 else before) + q, q))
        if rng.random() < 0.3:
            segs.append((int(rng.choice([1, 33, 900])), 1))
        dtype = torch.bfloat16 if rng.random() < 0.7 else torch.float32
        out, ref = kernel_cases._paged_case(ops, dtype, segs, nh, nkv, dh, page, window, seed=100 * block + trial,
                                            ws=ws if rng.random() < 0.8 else None)
        err = kernel_cases.rel(out, ref)
        assert err < kernel_cases.tol(dtype, 3e-6, 1.5e-2), (
            f"block {block} trial {trial}: {dtype} heads {nh}/{nkv}/{dh} page {page} window {window} "
            f"(context, tokens) {segs}: {err}")


ROWS = [1, 2, 7, 8, 12, 13, 16, 17, 31, 32, 33, 48, 64, 65, 100, 127, 128, 129, 200, 256, 257, 384, 385, 512, 700, 1000,
        1024, 1100, 2048, 2100]
COLUMNS = [16, 37, 64, 100, 128, 200, 224, 288, 301, 512, 1000, 1536, 2500, 3584, 4608, 4793, 6627, 9001]
DEPTHS = [8, 16, 40, 64, 72, 96, 128, 192, 256, 264, 320, 512, 1160]


@pytest.mark.parametrize("block", range(2))
def test_random_products_match_numpy(ops, block):
    """x w^T at random sizes on both sides of every rule that picks a kernel or a tiling (rows, columns, K a
    multiple of 64 or not, with and without lent memory for K in parts), with bias, into a float32 sum, and with
    the SwiGLU epilogue."""
    import math
    import plain_impl
    rng = np.random.default_rng(3 + block)
    for trial in range(80):
        m, n, k = int(rng.choice(ROWS)), int(rng.choice(COLUMNS)), int(rng.choice(DEPTHS))
        if rng.random() < 0.1:
            k = int(rng.choice([4, 36, 100, 90]))
        dtype = torch.bfloat16 if rng.random() < 0.7 else torch.float32
        swiglu = dtype is torch.bfloat16 and rng.random() < 0.33 and ops.swiglu_takes(m, k, dtype)
        g = torch.Generator().manual_seed(1000 * block + trial)
        ws = kernel_cases._Lender() if rng.random() < 0.7 else None
        if swiglu:
            n = min(n, 4800)
            x = (torch.randn(m, k, generator=g) * 2).to(dtype)
            w = (torch.randn(2 * n, k, generator=g) / math.sqrt(k)).to(dtype)
            y = x.double().numpy() @ w.double().numpy().T
            ref = plain_impl.swiglu(y[:, :n], y[:, n:])
            out = torch.full((m, n), float("nan"), dtype=dtype, device="cuda:0")
            ops.linear_swiglu(x.to("cuda:0"), w.to("cuda:0"), out)
            limit, what = 5e-3, f"with SwiGLU {m} x {n} x {k}"
        else:
            bias, acc = bool(rng.random() < 0.5), bool(rng.random() < 0.4)
            x = torch.randn(m, k, generator=g).to(dtype)
            w = (torch.randn(n, k, generator=g) / math.sqrt(k)).to(dtype)
            b = torch.randn(n, generator=g) if bias else None
            ref = plain_impl.linear(x.double().numpy(), w.double().numpy(), None if b is None else b.double().numpy())
            if acc:
                base = torch.randn(m, n, generator=g)
                out = base.to("cuda:0")
                ref = ref + base.double().numpy()
            else:
                wide = dtype is torch.float32 or rng.random() < 0.3
                out = torch.full((m, n), float("nan"), dtype=torch.float32 if wide else dtype, device="cuda:0")
            ops.linear(x.to("cuda:0"), w.to("cuda:0"), None if b is None else b.to("cuda:0"), out, accumulate=acc, ws=ws)
            limit = 4 * math.sqrt(k) * 2.0 ** -24 if out.dtype is torch.float32 else 5e-3
            what = f"{dtype} {m} x {n} x {k}, bias {bias}, into a sum {acc}, out {out.dtype}, lent memory {ws is not None}"
        err = kernel_cases.rel(out, ref)
        assert err < limit, f"block {block} trial {trial}: {what}: {err}"


@pytest.mark.parametrize("name", list(CASES))
def test_the_scheduler_with_random_budgets_and_pools_gives_the_plain_greedy_tokens(tmp_path, name):
    """Random prompts and limits, portions of 4 to 33 tokens, budgets of one to three portions, 2 to 8 slots, a
    pool that just holds the largest request, twice that or plenty (so that some runs preempt), steps started
    ahead or not; float32, where a request's greedy tokens are the plain implementation's."""
    import plain_impl
    from litinfer_amd.engine import Engine, Scheduler
    cfg, page, seed = CASES[name]
    d = helpers.make_model(tmp_path, cfg, seed)
    pcfg, weights = plain_impl.load_folder(d)
    preempted = 0
    for trial in range(8):
        rng = np.random.default_rng(100 * trial + seed)
        n = int(rng.integers(3, 9))
        lens = [min(int(x), int(cfg["max_position_embeddings"]) - 12) for x in rng.choice([1, 2, 7, 16, 17, 33, 40, 64, 90], n)]
        prompts = list(helpers.random_requests(cfg["vocab_size"], lens, 50 + trial).values())
        limits = [int(x) for x in rng.choice([1, 2, 5, 9, 12], n)]
        need = max(-(-(a + b) // page) * page for a, b in zip(lens, limits))
        pool = int(rng.choice([need + page, 2 * need, 4096]))
        portion = int(rng.choice([4, 8, 16, 33]))
        eng = Engine.from_dir(d, dtype="float32", device="cuda:0", page_size=page, max_tokens=pool,
                              max_seqs=int(rng.choice([2, 4, 8])))
        s = Scheduler(eng, eos_token_ids=(), chunk_size=portion, max_batch_tokens=portion * int(rng.choice([1, 2, 3])),
                      lookahead=bool(rng.random() < 0.5))
        ids = [s.add_request(p, m) for p, m in zip(prompts, limits)]
        while s.has_unfinished():
            s.step()
            assert s.steps < 5000, "the scheduler does not come to an end"
        eng.cache.check_invariants()
        assert all(f == g.pool.capacity for f, g in zip(eng.cache.free_pages(), eng.cache.groups))
        for i, p, m in zip(ids, prompts, limits):
            assert s.output(i) == plain_impl.greedy_generate(pcfg, weights, p, m), (name, trial, len(p), m, pool, portion)
        preempted += s.preemptions
    print(f"[observed] {name}: {preempted} preemptions over 8 runs")
