"""The engine's parts and paths, each on its own: on the CPU with the torch
stand-ins of tests/torch_ops.py (bookkeeping), and on the GPU with the HIP
kernels (`-m gpu`).  Compared with the plain implementation."""
import math
from dataclasses import dataclass, replace

import numpy as np
import pytest
import torch

import helpers
import plain_impl as P
import schedules
from litinfer_amd.cache import CacheFull, CacheManager
from litinfer_amd.config import ExecEntry, LayerSpec, ModelSpec, PartSpec, Qwen2Config, qwen2_model_spec, register_architecture
from litinfer_amd.engine import Engine, StepEntry, StepError
from litinfer_amd.engine.batch import BatchUploader, build_context
from litinfer_amd.engine.workspace import Workspace
from litinfer_amd.parts import (BatchNeeds, FeedForward, Mixer, PagedNeed, PagedTensor, Position, ResidualStream, Runtime,
                                StateNeed, build_part, register_part)
from litinfer_amd.weights import ParamSpec
from tiny_configs import TINY_A, TINY_B, TINY_C, TINY_E
from toy_parts import ToyConfig


@pytest.fixture(params=[pytest.param("cpu"), pytest.param("gpu", marks=pytest.mark.gpu)])
def device(request):
    if request.param == "cpu":
        request.getfixturevalue("cpu_ops")
        return "cpu"
    return "cuda:0"


F32_TOL, BF16_TOL = 2e-5, 1.5e-2


def engine_for(d, device, dtype="float32", page=16, max_tokens=512, **kw):
    return Engine.from_dir(d, dtype=dtype, device=device, page_size=page, max_tokens=max_tokens, max_seqs=4, **kw)


# ------------------------------------------------------------- whole paths
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_rolls_the_window_and_matches(tmp_path, device, dtype):
    if device == "cpu" and dtype == "bfloat16":
        pytest.skip("the stand-ins check bookkeeping; once is enough")
    stored = torch.float32 if dtype == "float32" else torch.bfloat16
    d = helpers.make_model(tmp_path, TINY_B, 1, stored)
    toks = helpers.random_requests(320, [250], 5)["r0"]
    ref = helpers.plain_logits(d, {"r0": toks})["r0"]
    eng = engine_for(d, device, dtype=dtype, page=8, max_tokens=256)
    rows = [eng.step([StepEntry("r0", toks[:3], [0, 1, 2])]).cpu().numpy()]
    for t in toks[3:]:
        rows.append(eng.step([StepEntry("r0", [t], [0])]).cpu().numpy())
    assert schedules.rel_err(np.concatenate(rows), ref) < (F32_TOL if dtype == "float32" else BF16_TOL)
    assert eng.cache.groups[1].pool.used <= 32 // 8 + 1          # the windowed layers keep a few pages only
    assert eng.cache.groups[0].pool.used == -(-250 // 8)


def test_a_short_portion_behind_a_long_cached_part(tmp_path, device):
    if device == "cpu":
        pytest.skip("a matter of the attention kernels' choice of runs")
    # few tiles of queries against some thousand keys: the attention of such a step cuts every tile's keys
    # into runs over several blocks and joins them; through the engine, against the plain implementation
    cfg = dict(TINY_E, max_position_embeddings=2304)
    d = helpers.make_model(tmp_path, cfg, 3, torch.bfloat16)
    toks = helpers.random_requests(cfg["vocab_size"], [2250], 9)["r0"]
    ref = helpers.plain_logits(d, {"r0": toks})["r0"]
    eng = engine_for(d, device, dtype="bfloat16", page=32, max_tokens=2304)
    eng.step([StepEntry("r0", toks[:2048], [])])
    rows = [eng.step([StepEntry("r0", toks[2048:2148], list(range(100)))]).cpu().numpy(),       # 4 tiles behind 2,048
            eng.step([StepEntry("r0", toks[2148:2150], [0, 1])]).cpu().numpy(),                 # down to two tokens
            eng.step([StepEntry("r0", toks[2150:], list(range(100)))]).cpu().numpy()]
    assert schedules.rel_err(np.concatenate(rows), ref[2048:]) < BF16_TOL


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_of_a_sequence(tmp_path, device, dtype):
    if device == "cpu" and dtype == "bfloat16":
        pytest.skip("the stand-ins check bookkeeping; once is enough")
    d = helpers.make_model(tmp_path, TINY_C, 2, torch.float32 if dtype == "float32" else torch.bfloat16)
    for n in (1, 2, 3):
        toks = helpers.random_requests(301, [n], n)["r0"]
        ref = helpers.plain_logits(d, {"r0": toks})["r0"]
        eng = engine_for(d, device, dtype=dtype)
        got = eng.step([StepEntry("x", toks, list(range(n)))]).cpu().numpy()
        assert schedules.rel_err(got, ref) < (F32_TOL if dtype == "float32" else BF16_TOL)
        # one token at a time gives the same
        eng.finish("x")
        rows = [eng.step([StepEntry("y", [t], [0])]).cpu().numpy() for t in toks]
        assert schedules.rel_err(np.concatenate(rows), ref) < (F32_TOL if dtype == "float32" else BF16_TOL)


def test_greedy_generation_through_the_entry_point(tmp_path, device):
    from litinfer_amd.models import Qwen2, load
    for cfg, seed in ((TINY_A, 0), (TINY_B, 1)):
        d = helpers.make_model(tmp_path / str(seed), cfg, seed)
        pcfg, w = P.load_folder(d)
        model = load(d, device=device, dtype="float32", max_tokens=512, max_seqs=4, chunk_size=24)
        assert isinstance(model, Qwen2)
        for n in (5, 17, 33):
            prompt = helpers.random_requests(cfg["vocab_size"], [n], n)["r0"]
            got = model.generate(prompt, max_new_tokens=16)
            assert got == P.greedy_generate(pcfg, w, prompt, 16, eos=cfg.get("eos_token_id", []) or [])
        assert model.generate(prompt) == got[:1]                       # max_new_tokens=None means one token
        assert model.generate(prompt, max_new_tokens=0) == []
        with pytest.raises(ValueError, match="max sequence length"):
            model.generate([1] * (cfg["max_position_embeddings"] + 1))   # test/test_kv_cache.py:87-93
        with pytest.raises(ValueError, match="must not be empty"):
            model.generate([])
        assert model.generate(prompt, max_new_tokens=16) == got          # the cache was given back in between
        assert model.engine.cache.free_slots() == 4


def test_continuous_batching_calls_give_each_request_its_own_greedy_tokens(tmp_path, device):
    from litinfer_amd.models import Qwen2
    d = helpers.make_model(tmp_path, TINY_A, 0)
    pcfg, w = P.load_folder(d)
    model = Qwen2(d, device=device, dtype="float32", max_tokens=256, max_seqs=4, chunk_size=8, max_batch_tokens=16)
    prompts = list(helpers.random_requests(256, [5, 17, 33], 9).values())
    model.engine_start()
    ids = [model.engine_add_request(p, max_new_tokens=6) for p in prompts]
    finished = 0
    while model.engine_has_unfinished():
        finished += model.engine_step()
    assert finished == 3 and model.engine_num_seqs() == 3
    for i, p in zip(ids, prompts):
        assert model.engine_is_finished(i) and model.engine_get_output(i) == P.greedy_generate(pcfg, w, p, 6)
    model.engine_stop()


def test_seeded_sampling_does_not_depend_on_the_batch(tmp_path, device):
    from litinfer_amd.engine import Scheduler
    from litinfer_amd.sampling import SamplingParams
    d = helpers.make_model(tmp_path, TINY_B, 1)
    prompts = list(helpers.random_requests(320, [1, 16, 40, 100], 3).values())
    params = [SamplingParams(temperature=0.8, seed=s) for s in range(4)]

    def run(which, **kw):
        eng = engine_for(d, device, page=8, max_tokens=1024)
        s = Scheduler(eng, eos_token_ids=(), **kw)
        ids = [s.add_request(prompts[i], 24, params[i]) for i in which]
        s.run_to_completion()
        return [s.output(i) for i in ids]
    together = run(range(4), chunk_size=24, max_batch_tokens=48)
    alone = [run([i])[0] for i in range(4)]
    assert together == alone and all(len(t) == 24 for t in together)
    assert len({tuple(t) for t in together}) == 4


def test_the_sampling_table_on_the_device_gives_the_tokens_of_options_sent_with_every_step(tmp_path, device):
    """The scheduler's own sampler keeps every live request's options, seed and count of draws in a table on
    the device, a row per state slot, written once when the request first samples in its slot; each step
    then sends the rows' slots only.  Same tokens as a sampler that is sent options and uniform numbers with
    every step: with large and negative seeds, top-k and top-p, greedy requests in between, the first token
    forced greedy, and with so few pages that requests are preempted and later go on in another slot."""
    from litinfer_amd.engine import Scheduler
    from litinfer_amd.sampling import Sampler, SamplingParams
    d = helpers.make_model(tmp_path, TINY_B, 1)
    prompts = list(helpers.random_requests(320, [3, 30, 70, 9, 41, 18], 21).values())
    params = [SamplingParams(temperature=0.9, top_k=40, seed=2 ** 63 + 12345), None,
              SamplingParams(temperature=1.3, top_p=0.8, seed=-7), SamplingParams(temperature=0.7, seed=3),
              SamplingParams(), SamplingParams(temperature=1.0, top_k=5, top_p=0.9, seed=2 ** 40)]

    def run(table, max_tokens, lookahead):
        eng = engine_for(d, device, page=8, max_tokens=max_tokens)
        sampler = Sampler(eng.rt.device, slots=eng.cache.max_seqs if table else 0)
        s = Scheduler(eng, eos_token_ids=(), chunk_size=16, max_batch_tokens=40, lookahead=lookahead, sampler=sampler)
        ids = [s.add_request(p, 20, sp, first_token_greedy=i % 2 == 0) for i, (p, sp) in enumerate(zip(prompts, params))]
        s.run_to_completion()
        eng.cache.check_invariants()
        return [s.output(i) for i in ids], s.preemptions, sampler
    want, pre, _ = run(False, 1024, False)
    assert pre == 0 and all(len(t) == 20 for t in want)
    got, pre, sampler = run(True, 1024, True)
    assert got == want and pre == 0
    assert sampler.table is not None and int(sampler.table[:, 5].max()) >= 19          # draws were counted on the device
    got, pre, _ = run(True, 136, True)
    assert got == want and pre > 0
    got, pre, _ = run(True, 136, False)
    assert got == want and pre > 0


def test_step_refuses_bad_batches_and_leaves_the_cache_alone(tmp_path, device):
    d = helpers.make_model(tmp_path, TINY_A, 0)
    eng = engine_for(d, device, max_tokens=64)
    eng.step([StepEntry("a", [1, 2, 3], [])])
    before = (eng.cache.free_pages(), eng.cache.cached_len("a"))
    for bad in ([], [StepEntry("a", [], [])], [StepEntry("a", [256], [0])], [StepEntry("a", [-1], [0])],
                [StepEntry("a", [1], [1])], [StepEntry("a", [1], []), StepEntry("a", [2], [])],
                [StepEntry("b", [1] * 129, [])]):
        with pytest.raises(StepError):
            eng.step(bad)
    with pytest.raises(CacheFull):
        eng.step([StepEntry("a", [1], []), StepEntry("c", [1] * 60, [])])
    assert (eng.cache.free_pages(), eng.cache.cached_len("a")) == before and not eng.cache.has("c")
    assert eng.step([StepEntry("a", [4], [])]) is None                 # nothing wanted: nothing returned
    eng.finish("a")
    eng.finish("a")                                                    # ending twice is harmless
    assert eng.cache.free_pages() == [4]


@pytest.mark.parametrize("stored", [torch.float32, torch.float16])
def test_matrices_are_bound_in_the_engines_dtype_whatever_the_checkpoint_stores(tmp_path, device, stored, capsys):
    """A bfloat16 engine rounds matrices stored in 32-bit or half precision once to bfloat16 (every
    product then takes the bfloat16 kernels) and says so in one line; norm weights and biases stay
    32-bit; `keep_stored_precision` keeps the matrices in 32-bit; a 32-bit engine widens everything."""
    d = helpers.make_model(tmp_path, TINY_A, 0, stored)
    toks = helpers.random_requests(256, [40], 1)["r0"]
    rounded = helpers.plain_logits(d, {"r0": toks}, matrices_as_bfloat16=True)["r0"]
    as_stored = helpers.plain_logits(d, {"r0": toks})["r0"]
    assert schedules.rel_err(rounded, as_stored) > 1e-4          # the two references can be told apart
    eng = engine_for(d, device, dtype="bfloat16")
    notes = [l for l in capsys.readouterr().err.splitlines() if "rounded once" in l]
    assert len(notes) == 1 and ("F32" if stored is torch.float32 else "F16") in notes[0]
    mixer, ffn = eng.model.layers[0].mixer, eng.model.layers[0].ffn
    for w in (mixer.qkv.weight, mixer.out.weight, ffn.gate_up.weight, ffn.down.weight, eng.model.embedding.table,
              eng.model.head.proj.weight):
        assert w.dtype is torch.bfloat16
    assert mixer.qkv.bias.dtype is torch.float32 and eng.model.layers[0].norm1.weight.dtype is torch.float32
    want = torch.from_numpy(helpers.round_to_bfloat16(
        helpers.plain_impl.load_folder(d, np.float32)[1]["model.layers.0.mlp.down_proj.weight"]))
    assert torch.equal(ffn.down.weight.float().cpu(), want)     # the engine's rounding is nearest-even, once
    out = eng.step([StepEntry("a", toks, list(range(40)))]).cpu().numpy()
    assert schedules.rel_err(out, rounded) < BF16_TOL
    kept = engine_for(d, device, dtype="bfloat16", keep_stored_precision=True)
    assert not [l for l in capsys.readouterr().err.splitlines() if "rounded once" in l]
    assert kept.model.layers[0].mixer.qkv.weight.dtype is torch.float32
    out = kept.step([StepEntry("a", toks, list(range(40)))]).cpu().numpy()
    assert schedules.rel_err(out, as_stored) < BF16_TOL
    wide = engine_for(d, device, dtype="float32")
    assert wide.model.layers[0].mixer.qkv.weight.dtype is torch.float32
    out = wide.step([StepEntry("a", toks, list(range(40)))]).cpu().numpy()
    assert schedules.rel_err(out, as_stored) < F32_TOL


# ------------------------------------------------------ each part on its own
def _rt(device, dtype=torch.float32):
    return Runtime(torch.device(device), dtype)


def _load(part, tensors):
    part.load_params(lambda name: tensors.get(name))
    return part


def test_norm_part_alone(device):
    g = torch.Generator().manual_seed(0)
    x, w = torch.randn(9, 120, generator=g), 1 + 0.1 * torch.randn(120, generator=g)
    part = _load(build_part("norm", PartSpec("rmsnorm", "n.", {"size": 120, "eps": 1e-4}), _rt(device)), {"n.weight": w})
    assert part.expected_params() == {"n.weight": ParamSpec((120,), init="one_plus_normal")}
    out = torch.empty(9, 120, device=device)
    part.forward(x.to(device), out)
    assert schedules.rel_err(out.cpu().numpy(), P.rms_norm(x.double().numpy(), w.double().numpy(), 1e-4)) < 2e-6


def test_feed_forward_part_alone(device):
    g = torch.Generator().manual_seed(1)
    h, i, t = 72, 200, 11
    ws = {f"f.{n}_proj.weight": torch.randn(*s, generator=g) * 0.1 for n, s in
          (("gate", (i, h)), ("up", (i, h)), ("down", (h, i)))}
    part = _load(build_part("feed_forward", PartSpec("swiglu_mlp", "f.", {"hidden_size": h, "intermediate_size": i}),
                            _rt(device)), ws)
    x = torch.randn(t, h, generator=g)
    res = torch.randn(t, h, generator=g)
    out = res.clone().to(device)
    ctx = type("Ctx", (), {"ws": Workspace(device)})()
    part.forward(x.to(device), ResidualStream(out, ctx.ws), ctx)
    xd = x.double().numpy()
    d = {k: v.double().numpy() for k, v in ws.items()}
    ref = res.double().numpy() + P.swiglu(xd @ d["f.gate_proj.weight"].T, xd @ d["f.up_proj.weight"].T) @ d["f.down_proj.weight"].T
    assert schedules.rel_err(out.cpu().numpy(), ref) < 2e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_norm_shared_through_the_stream(device, dtype):
    """The product before a norm may leave the rows that the part behind the norm
    multiplies; any other write to the stream forgets them; a part that knows nothing
    of this gets the norm as a pass of its own.  The result is the same either way."""
    from litinfer_amd.parts.linear import Linear
    g = torch.Generator().manual_seed(3)
    h, i, k, t = 72, 200, 40, 5
    rt = _rt(device, dtype)
    stored = lambda x: x.to(dtype)
    ws = {f"f.{n}_proj.weight": stored(torch.randn(*s, generator=g) * 0.1) for n, s in
          (("gate", (i, h)), ("up", (i, h)), ("down", (h, i)))}
    gamma = 1 + 0.1 * torch.randn(h, generator=g)
    ffn = _load(build_part("feed_forward", PartSpec("swiglu_mlp", "f.", {"hidden_size": h, "intermediate_size": i}), rt), ws)
    norm = _load(build_part("norm", PartSpec("rmsnorm", "n.", {"size": h, "eps": 1e-5}), rt), {"n.weight": gamma})
    other = _load(build_part("norm", PartSpec("rmsnorm", "o.", {"size": h, "eps": 1e-5}), rt), {"o.weight": gamma})
    wprev = stored(torch.randn(h, k, generator=g) * 0.2)
    prev = Linear(rt, wprev)
    hp = stored(torch.randn(t, k, generator=g))
    res = torch.randn(t, h, generator=g) * torch.logspace(-1, 1, t)[:, None]
    x1 = res.double().numpy() + hp.double().numpy() @ wprev.double().numpy().T
    d = {n: v.double().numpy() for n, v in ws.items()}
    xn = P.rms_norm(x1, gamma.double().numpy(), 1e-5)
    ref = x1 + P.swiglu(xn @ d["f.gate_proj.weight"].T, xn @ d["f.up_proj.weight"].T) @ d["f.down_proj.weight"].T
    outs = []
    for announce in (True, False):
        ctx = type("Ctx", (), {"ws": Workspace(device)})()
        stream = ResidualStream(res.clone().to(device), ctx.ws)
        stream.next_norm = norm if announce else None
        stream.add_linear(prev, hp.to(device))
        left = stream.scaled_rows(norm)
        assert (left is not None) == (announce and dtype is torch.bfloat16)       # few bfloat16 rows: the kernels take it
        assert stream.scaled_rows(other) is None                                     # another norm's reader finds nothing
        buf = torch.empty(t, h, dtype=dtype, device=device)
        ffn.forward_prenorm(norm, stream, buf, ctx)
        outs.append(stream.tensor().cpu().numpy())
        assert schedules.rel_err(outs[-1], ref) < (F32_TOL if dtype is torch.float32 else BF16_TOL)
    # whoever takes the sum itself may write to it: what was left for the norm is forgotten
    ctx = type("Ctx", (), {"ws": Workspace(device)})()
    stream = ResidualStream(res.clone().to(device), ctx.ws)
    stream.next_norm = norm
    stream.add_linear(prev, hp.to(device))
    stream.tensor()
    assert stream.scaled_rows(norm) is None
    stream.next_norm = norm
    stream.add_linear(prev, hp.to(device))
    stream.next_norm = None
    stream.add_linear(prev, hp.to(device))                       # a second addition, with no reader announced
    assert stream.scaled_rows(norm) is None


def _mixer_case(device, window, cache_steps):
    """Run the attention mixer alone over two requests in several steps and
    return (its additions to a zero residual, the plain result)."""
    g = torch.Generator().manual_seed(2)
    h, nh, nkv, dh, page = 40, 6, 2, 16, 4
    args = {"hidden_size": h, "num_heads": nh, "num_kv_heads": nkv, "head_dim": dh, "qkv_bias": True,
            "window": window, "scale": None,
            "position": PartSpec("rope_neox", "", {"head_dim": dh, "rotary_dim": dh, "theta": 1e4})}
    ws = {f"a.{n}_proj.weight": torch.randn(o, h, generator=g) * 0.2 for n, o in (("q", nh * dh), ("k", nkv * dh), ("v", nkv * dh))}
    ws.update({f"a.{n}_proj.bias": torch.randn(o, generator=g) * 0.2 for n, o in (("q", nh * dh), ("k", nkv * dh), ("v", nkv * dh))})
    ws["a.o_proj.weight"] = torch.randn(h, nh * dh, generator=g) * 0.2
    mixer = _load(build_part("mixer", PartSpec("gqa_attention", "a.", args), _rt(device)), ws)
    cache = CacheManager([mixer.cache_need()], [None], page_size=page, num_pages=16, max_seqs=2,
                         dtype=torch.float32, device=device, page_order_seed=3)
    xs = {"p": torch.randn(19, h, generator=g), "q": torch.randn(7, h, generator=g)}
    wsp, up = Workspace(device), BatchUploader(device)
    got = {k: [] for k in xs}
    done = {k: 0 for k in xs}
    for step in cache_steps:
        entries = [StepEntry(r, [0] * n, []) for r, n in step]
        for e in entries:
            if not cache.has(e.rid):
                cache.admit(e.rid)
            cache.reserve(e.rid, len(e.tokens))
        ctx = build_context(cache, entries, wsp, up)
        x = torch.cat([xs[r][done[r]:done[r] + n] for r, n in step]).to(device)
        res = torch.zeros(x.shape[0], h, device=device)
        mixer.forward(x, ResidualStream(res, wsp), ctx, cache.view(0))
        o = 0
        for r, n in step:
            got[r].append(res[o:o + n].cpu().numpy())
            cache.commit(r, n)
            done[r] += n
            o += n
    d = {k: v.double().numpy() for k, v in ws.items()}
    ref = {}
    for r, x in xs.items():
        xd, t = x.double().numpy(), x.shape[0]
        q = P.rope_neox((xd @ d["a.q_proj.weight"].T + d["a.q_proj.bias"]).reshape(t, nh, dh), np.arange(t), 1e4)
        k = P.rope_neox((xd @ d["a.k_proj.weight"].T + d["a.k_proj.bias"]).reshape(t, nkv, dh), np.arange(t), 1e4)
        v = (xd @ d["a.v_proj.weight"].T + d["a.v_proj.bias"]).reshape(t, nkv, dh)
        a = P.attention(q, k, v, np.arange(t), np.arange(t), 1 / math.sqrt(dh), window)
        ref[r] = a.reshape(t, -1) @ d["a.o_proj.weight"].T
    return {r: np.concatenate(v) for r, v in got.items()}, ref


@pytest.mark.parametrize("window", [0, 5])
def test_attention_mixer_alone_over_a_cut_up_batch(device, window):
    steps = [[("p", 6)], [("p", 2), ("q", 3)], [("p", 1), ("q", 1)], [("q", 3), ("p", 10)]]
    got, ref = _mixer_case(device, window, steps)
    for r in ref:
        assert schedules.rel_err(got[r], ref[r]) < 3e-6


def test_position_part_alone(device):
    g = torch.Generator().manual_seed(4)
    part = build_part("position", PartSpec("rope_neox", "", {"head_dim": 24, "rotary_dim": 24, "theta": 5e4}), _rt(device))
    x = torch.randn(5, 3 * 24, generator=g)
    pos = np.array([0, 1, 7, 8, 100], dtype=np.int32)
    ctx = type("Ctx", (), {})()
    ctx.ws, ctx.num_tokens, ctx.positions, ctx._s = Workspace(device), 5, torch.from_numpy(pos).to(device), {}
    ctx.shared = lambda key, make: ctx._s.setdefault(key, make())
    xd = x.clone().to(device)
    part.apply(xd, 3, 24, ctx)
    ref = P.rope_neox(x.double().numpy().reshape(5, 3, 24), pos, 5e4).reshape(5, -1)
    assert schedules.rel_err(xd.cpu().numpy(), ref) < 1e-5
    with pytest.raises(ValueError):
        build_part("position", PartSpec("rope_neox", "", {"head_dim": 24, "rotary_dim": 26, "theta": 1.0}), _rt(device))
    with pytest.raises(KeyError, match="registered: .*rope_neox"):
        build_part("position", PartSpec("nope"), _rt(device))


def test_embedding_and_head_alone(device):
    g = torch.Generator().manual_seed(5)
    table = torch.randn(301, 56, generator=g)
    emb = _load(build_part("embedding", PartSpec("token_embedding", "e.", {"vocab_size": 301, "hidden_size": 56}),
                           _rt(device)), {"e.weight": table})
    ids = torch.tensor([300, 0, 7, 7], dtype=torch.int32)
    out = torch.empty(4, 56, device=device)
    emb.forward(ids.to(device), out)
    assert torch.equal(out.cpu(), table[ids.long()])
    head = build_part("head", PartSpec("linear_head", "h.", {"vocab_size": 301, "hidden_size": 56, "tied_to": "e.weight"}),
                      _rt(device))
    head.load_params(lambda n: None, tied_table=emb.table)
    assert head.expected_params() == {}
    logits = torch.empty(4, 301, device=device)
    head.forward(out, logits, Workspace(device))
    assert schedules.rel_err(logits.cpu().numpy(), (table[ids.long()] @ table.T).double().numpy()) < 2e-6


# ------------------------------------- the order of layers is data: twice, shared cache
def _looped_spec(c: Qwen2Config) -> ModelSpec:
    base = qwen2_model_spec(c)
    return replace(base, architecture="LoopedQwen2Test",
                   order=(ExecEntry(0), ExecEntry(1), ExecEntry(0), ExecEntry(1, cache_from=1)))


register_architecture("LoopedQwen2Test", Qwen2Config.from_dict, _looped_spec)


def test_a_layer_named_twice_and_a_layer_reading_anothers_cache(tmp_path, device):
    cfg = dict(TINY_A, architectures=["LoopedQwen2Test"])
    d = helpers.make_model(tmp_path, cfg, 3)
    pcfg, w = P.load_folder(d)
    reqs = helpers.random_requests(256, [37, 9], 4)
    order = [(0, None), (1, None), (0, None), (1, 1)]
    ref = {r: P.forward(pcfg, w, t, order=order) for r, t in reqs.items()}
    eng = engine_for(d, device)
    assert len(eng.cache.groups) == 1 and eng.cache.groups[0].entries == [0, 1, 2]   # three caches, four entries
    for kind in ("whole", "chunks", "mixed"):
        out = schedules.run(eng, reqs, getattr(schedules, kind)(reqs))
        assert max(schedules.rel_err(out[r], ref[r]) for r in reqs) < F32_TOL, kind


# ------------------------------ a toy mixer with state of its own, defined in tests/toy_parts.py
def test_a_toy_mixer_with_state_is_registered_built_and_stepped(tmp_path, device):
    import toy_parts                                       # registers the part and the architecture
    cfg = dict(TINY_A, architectures=["ToyStateLM"], toy_decay=0.9)
    d = helpers.make_model(tmp_path, cfg, 6)
    pcfg, w = P.load_folder(d)
    assert "model.layers.0.toy.w" in w and "model.layers.0.self_attn.q_proj.weight" not in w
    assert not w["model.layers.0.toy.b"].any()             # the part said "zeros" of its bias
    reqs = helpers.random_requests(256, [21, 40, 3, 30, 12], 7)
    ref = {r: toy_parts.plain_toy_state_logits(pcfg, w, t, 0.9) for r, t in reqs.items()}
    eng = engine_for(d, device)
    assert len(eng.cache.groups) == 1 and eng.cache.groups[0].entries == [1]
    assert eng.cache.view(0).state.shape == (4, 64)
    for kind in ("whole", "tail", "chunks", "mixed"):
        out = schedules.run(eng, reqs, getattr(schedules, kind)(reqs))
        assert max(schedules.rel_err(out[r], ref[r]) for r in reqs) < F32_TOL, kind   # slots reused, state zeroed
    eng.cache.check_invariants()


def test_a_toy_mixer_keeps_pages_and_a_state_of_fixed_size(tmp_path, device):
    """Keys and values in pages beside a tail of the last three inputs in the request's state slot
    (tests/toy_parts.py): one mixer, both kinds of cache, no framework file touched.  The toy's
    pages form a group of their own beside the attention layer's; slots and pages are used again."""
    import toy_parts
    cfg = dict(TINY_A, architectures=["ToyTailLM"], toy_decay=0.0)
    d = helpers.make_model(tmp_path, cfg, 16)
    pcfg, w = P.load_folder(d)
    assert "model.layers.0.tail.wk" in w and "model.layers.0.self_attn.q_proj.weight" not in w
    reqs = helpers.random_requests(256, [21, 40, 3, 30, 12, 1, 2], 17)
    ref = {r: toy_parts.plain_toy_tail_logits(pcfg, w, t) for r, t in reqs.items()}
    for kind in ("whole", "tail", "chunks", "mixed"):
        steps = getattr(schedules, kind)(reqs)
        eng = engine_for(d, device, page=8, max_tokens=schedules.max_live_tokens(reqs, steps, 8 if kind == "mixed" else 64),
                         page_order_seed=5)
        assert [g.entries for g in eng.cache.groups] == [[0], [1]] and set(eng.cache.groups[0].data) == {"k", "v"}
        v = eng.cache.view(0)
        assert v.tensors["k"].shape[1:] == (8, 12) and v.states["tail"].shape == (4, 3, 64) and v.state is v.states["tail"]
        out = schedules.run(eng, reqs, steps)
        assert max(schedules.rel_err(out[r], ref[r]) for r in reqs) < F32_TOL, kind
        eng.cache.check_invariants()
        if kind == "mixed":
            assert all(g.pool.total_allocations > g.pool.capacity for g in eng.cache.groups)


# ------------- a toy mixer with a cache of its own shape: one latent vector per token, in pages
class ToyLatentAttention(Mixer):
    """One head over a compressed cache: c_t = xn_t Wc (a latent of `rank` numbers, kept in
    pages as float32 under the name "c"), score(t, s) = (xn_t Wq) . c_s / sqrt(rank) for
    s <= t, y_t = softmax(score) c, output y_t Wo.  Neither keys nor values are stored.
    Written with torch: it is a toy that shows the interface, not a kernel."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.h, self.rank = spec.args["hidden_size"], spec.args["rank"]

    def cache_need(self):
        return PagedNeed((PagedTensor("c", (self.rank,), torch.float32),))

    def expected_params(self):
        p = self.prefix
        return {p + "wc": ParamSpec((self.rank, self.h)), p + "wq": ParamSpec((self.rank, self.h)),
                p + "wo": ParamSpec((self.h, self.rank))}

    def load_params(self, get):
        self.wc, self.wq, self.wo = (get(self.prefix + n).to(torch.float32).to(self.rt.device) for n in ("wc", "wq", "wo"))

    def forward(self, xn, residual, ctx, cache):
        x = xn.float()
        pages = cache.tensors["c"]                                     # [pages, page_size, rank]
        flat = pages.view(-1, self.rank)
        flat[ctx.slot_map(cache.group).long()] = x @ self.wc.T         # written before it is read, like keys
        q = x @ self.wq.T
        table = ctx.attention_meta(cache.group).block_table.cpu()
        out = residual.tensor()
        for s in range(ctx.num_segments):
            q0, n, have = int(ctx.host_q_start[s]), int(ctx.host_q_len[s]), int(ctx.host_ctx_len[s])
            blocks = table[s, :-(-have // cache.page_size)].long().to(pages.device)
            c = pages[blocks].reshape(-1, self.rank)[:have]            # the request's latents in order
            score = q[q0:q0 + n] @ c.T / math.sqrt(self.rank)
            pos = torch.arange(have - n, have, device=score.device)[:, None]
            score = score.masked_fill(torch.arange(have, device=score.device)[None, :] > pos, float("-inf"))
            out[q0:q0 + n] += torch.softmax(score, dim=-1) @ c @ self.wo.T


def _latent_spec(c: ToyConfig) -> ModelSpec:
    base = qwen2_model_spec(c.inner)
    layers = tuple(LayerSpec("prenorm", dict(l.parts, mixer=PartSpec("toy_latent", f"model.layers.{i}.lat.",
                                                                     {"hidden_size": c.hidden_size, "rank": 12})))
                   for i, l in enumerate(base.layers))
    return replace(base, architecture="ToyLatentLM", layers=layers)


def test_a_toy_mixer_keeps_one_latent_vector_per_token_in_pages(tmp_path, device):
    register_part("mixer", "toy_latent", ToyLatentAttention)
    register_architecture("ToyLatentLM", ToyConfig.from_dict, _latent_spec)
    cfg = dict(TINY_A, architectures=["ToyLatentLM"], toy_decay=0.0)
    d = helpers.make_model(tmp_path, cfg, 12)
    pcfg, w = P.load_folder(d)

    def plain(ids):
        x = P.embedding(ids, w["model.embed_tokens.weight"])
        for l in range(2):
            p = f"model.layers.{l}."
            xn = P.rms_norm(x, w[p + "input_layernorm.weight"], 1e-6)
            c, q = xn @ w[p + "lat.wc"].T, xn @ w[p + "lat.wq"].T
            score = q @ c.T / math.sqrt(12)
            score[np.triu_indices(len(ids), 1)] = -np.inf
            e = np.exp(score - score.max(-1, keepdims=True))
            x = x + (e / e.sum(-1, keepdims=True)) @ c @ w[p + "lat.wo"].T
            xn = P.rms_norm(x, w[p + "post_attention_layernorm.weight"], 1e-6)
            x = x + P.swiglu(xn @ w[p + "mlp.gate_proj.weight"].T, xn @ w[p + "mlp.up_proj.weight"].T) @ w[p + "mlp.down_proj.weight"].T
        return P.rms_norm(x, w["model.norm.weight"], 1e-6) @ w["model.embed_tokens.weight"].T

    reqs = helpers.random_requests(256, [33, 18, 5, 26, 47], 9)
    ref = {r: plain(np.asarray(t)) for r, t in reqs.items()}
    for kind in ("whole", "tail", "chunks", "mixed"):
        steps = getattr(schedules, kind)(reqs)
        eng = engine_for(d, device, page=8, max_tokens=schedules.max_live_tokens(reqs, steps, 8 if kind == "mixed" else 64),
                         page_order_seed=4)
        g = eng.cache.groups
        assert len(g) == 1 and set(g[0].data) == {"c"} and g[0].data["c"].shape[2:] == (8, 12)
        assert g[0].data["c"].dtype is torch.float32 and g[0].entries == [0, 1]
        needs = eng.model.batch_needs()
        assert (needs.tile_rows, needs.token_kinds) == (0, False)        # nobody here wants tiles or token lists laid out
        out = schedules.run(eng, reqs, steps)
        assert max(schedules.rel_err(out[r], ref[r]) for r in reqs) < F32_TOL, kind
        eng.cache.check_invariants()
    # the architecture's own model does ask for them, through its attention
    needs = engine_for(helpers.make_model(tmp_path / "a", TINY_A, 0), device).model.batch_needs()
    assert (needs.tile_rows, needs.token_kinds) == (32, True)
    # and its products say in which tiles they take a step's rows (the kernel library's number; none on the stand-ins)
    assert needs.row_tile == (64 if device != "cpu" else 1)


# --------- a toy feed-forward with routing and a toy position encoding, defined here
class ToyRoutedFFN(FeedForward):
    """y = W2_e relu(W1_e xn) with e = argmax(router xn), one expert per token.
    Written with torch: it is a toy that shows the interface, not a kernel."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.h, self.inner, self.experts = (spec.args[k] for k in ("hidden_size", "inner", "experts"))

    def expected_params(self):
        p = self.prefix
        out = {p + "router.weight": ParamSpec((self.experts, self.h))}
        for e in range(self.experts):
            out[p + f"experts.{e}.w1"] = ParamSpec((self.inner, self.h))
            out[p + f"experts.{e}.w2"] = ParamSpec((self.h, self.inner))
        return out

    def load_params(self, get):
        f = lambda n: get(self.prefix + n).to(torch.float32).to(self.rt.device)
        self.router = f("router.weight")
        self.w1 = torch.stack([f(f"experts.{e}.w1") for e in range(self.experts)])
        self.w2 = torch.stack([f(f"experts.{e}.w2") for e in range(self.experts)])

    def forward(self, xn, residual, ctx):
        x = xn.float()
        choice = torch.argmax(x @ self.router.T, dim=-1)               # router logits in 32-bit
        hidden = torch.relu(torch.einsum("th,tih->ti", x, self.w1[choice]))
        residual.tensor().add_(torch.einsum("ti,thi->th", hidden, self.w2[choice]))


class ToyPairRope(Position):
    """Rotary encoding over NEIGHBOURING pairs (2j, 2j+1), unlike the half-split
    pairing of the architecture: another position encoding behind the same interface."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.dh, self.theta = spec.args["head_dim"], spec.args["theta"]

    def key(self):
        return ("toy_pair_rope", self.dh, self.theta)

    def tables(self, ctx):
        def make():
            j = torch.arange(self.dh // 2, dtype=torch.float32, device=ctx.positions.device)
            ang = ctx.positions.float()[:, None] / (self.theta ** (2 * j / self.dh))
            return torch.cos(ang), torch.sin(ang)
        return ctx.shared(self.key(), make)

    def apply(self, qkv, n_heads_total, head_dim, ctx):
        cos, sin = self.tables(ctx)
        x = qkv[:, :n_heads_total * head_dim].float().reshape(qkv.shape[0], n_heads_total, head_dim // 2, 2)
        a, b = x[..., 0], x[..., 1]
        c, s = cos[:, None, :], sin[:, None, :]
        y = torch.stack([a * c - b * s, b * c + a * s], dim=-1).reshape(qkv.shape[0], -1)
        qkv[:, :n_heads_total * head_dim] = y.to(qkv.dtype)


def _routed_spec(c: ToyConfig) -> ModelSpec:
    base = qwen2_model_spec(c.inner)
    l0 = base.layers[0]
    mixer = l0.parts["mixer"]
    pair = PartSpec("toy_pair_rope", "", {"head_dim": c.inner.head_dim, "theta": c.inner.rope_theta})
    toy = LayerSpec("prenorm", dict(
        l0.parts,
        mixer=PartSpec(mixer.kind, mixer.prefix, dict(mixer.args, position=pair)),
        feed_forward=PartSpec("toy_routed", "model.layers.0.moe.",
                              {"hidden_size": c.hidden_size, "inner": 24, "experts": 3})))
    return replace(base, architecture="ToyRoutedLM", layers=(toy,) + base.layers[1:])


def test_a_toy_routed_feed_forward_and_another_position_encoding(tmp_path, device):
    register_part("feed_forward", "toy_routed", ToyRoutedFFN)
    register_part("position", "toy_pair_rope", ToyPairRope)
    register_architecture("ToyRoutedLM", ToyConfig.from_dict, _routed_spec)
    cfg = dict(TINY_A, architectures=["ToyRoutedLM"], toy_decay=0.0)
    d = helpers.make_model(tmp_path, cfg, 8)
    pcfg, w = P.load_folder(d)
    assert "model.layers.0.moe.experts.2.w2" in w and "model.layers.0.mlp.down_proj.weight" not in w
    nh, nkv, dh = pcfg["num_attention_heads"], pcfg["num_key_value_heads"], P.head_dim_of(pcfg)

    def pair_rope(x, pos, theta):
        j = np.arange(dh // 2)
        ang = np.asarray(pos, dtype=np.float64)[:, None] / (theta ** (2 * j / dh))
        c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
        a, b = x[..., 0::2], x[..., 1::2]
        y = np.empty_like(x)
        y[..., 0::2], y[..., 1::2] = a * c - b * s, b * c + a * s
        return y

    used = set()

    def plain(ids):
        t = len(ids)
        pos = np.arange(t)
        x = P.embedding(ids, w["model.embed_tokens.weight"])
        p = "model.layers.0."
        xn = P.rms_norm(x, w[p + "input_layernorm.weight"], 1e-6)
        proj = lambda n: P.linear(xn, w[p + f"self_attn.{n}_proj.weight"], w[p + f"self_attn.{n}_proj.bias"])
        q = pair_rope(proj("q").reshape(t, nh, dh), pos, pcfg["rope_theta"])
        k = pair_rope(proj("k").reshape(t, nkv, dh), pos, pcfg["rope_theta"])
        a = P.attention(q, k, proj("v").reshape(t, nkv, dh), pos, pos, 1 / math.sqrt(dh))
        x = x + P.linear(a.reshape(t, nh * dh), w[p + "self_attn.o_proj.weight"])
        xn = P.rms_norm(x, w[p + "post_attention_layernorm.weight"], 1e-6)
        choice = np.argmax(xn @ w[p + "moe.router.weight"].T, axis=-1)
        used.update(choice.tolist())
        y = np.stack([w[p + f"moe.experts.{e}.w2"] @ np.maximum(w[p + f"moe.experts.{e}.w1"] @ v, 0)
                      for e, v in zip(choice, xn)])
        x, _ = P.decoder_layer(x + y, pos, w, "model.layers.1.", pcfg, 0)
        return P.rms_norm(x, w["model.norm.weight"], 1e-6) @ w["model.embed_tokens.weight"].T

    reqs = helpers.random_requests(256, [33, 18, 5, 26], 9)
    ref = {r: plain(np.asarray(t)) for r, t in reqs.items()}
    assert len(used) > 1                                   # the router does choose
    eng = engine_for(d, device)
    for kind in ("whole", "tail", "chunks", "mixed"):
        out = schedules.run(eng, reqs, getattr(schedules, kind)(reqs))
        assert max(schedules.rel_err(out[r], ref[r]) for r in reqs) < F32_TOL, kind


# ----------------------------- tokens fed back on the device, steps started ahead
def test_an_entry_takes_its_token_from_the_feedback_buffer(tmp_path, device):
    d = helpers.make_model(tmp_path, TINY_A, 0)
    prompt = helpers.random_requests(256, [12], 5)["r0"]
    eng = engine_for(d, device)
    want = eng.step([StepEntry("a", prompt[:8], []), StepEntry("b", prompt, [11])]).clone()
    eng.finish("a"), eng.finish("b")
    # the same batch with three of the ids given through the buffer, beside wrong numbers in `tokens`
    eng.feedback[5], eng.feedback[9], eng.feedback[2] = prompt[7], prompt[0], prompt[11]
    a = StepEntry("a", prompt[:7] + [0], [], take=[-1] * 7 + [5])
    b = StepEntry("b", [1] + prompt[1:11] + [3], [11], take=[9] + [-1] * 10 + [2])
    got = eng.step([a, b])
    assert torch.equal(got, want)
    with pytest.raises(StepError):
        eng.step([StepEntry("c", [1, 2], [], take=[0])])          # one place for two tokens


@pytest.mark.parametrize("sampled", [False, True])
def test_steps_started_ahead_give_the_same_tokens(tmp_path, device, sampled):
    """The scheduler with lookahead against the one that waits for every token:
    end tokens (found out one step late), length limits, portions, preemption."""
    from litinfer_amd.engine import Scheduler
    from litinfer_amd.sampling import SamplingParams
    d = helpers.make_model(tmp_path, TINY_B, 1)
    prompts = list(helpers.random_requests(320, [3, 30, 70, 9, 41, 18], 13).values())
    limits = [40, 9, 25, 1, 33, 2]

    def run(lookahead, eos, max_tokens):
        eng = engine_for(d, device, page=8, max_tokens=max_tokens)
        s = Scheduler(eng, eos_token_ids=eos, chunk_size=16, max_batch_tokens=40, lookahead=lookahead)
        ids = [s.add_request(p, n, SamplingParams(temperature=0.9, top_k=50, seed=i) if sampled else None)
               for i, (p, n) in enumerate(zip(prompts, limits))]
        order = []
        while s.has_unfinished():
            order += s.step()
            assert s.steps < 2000, "the scheduler does not come to an end"
        eng.cache.check_invariants()
        assert all(f == g.pool.capacity for f, g in zip(eng.cache.free_pages(), eng.cache.groups))
        by_request = {i: [t for r, t in order if r == i] for i in ids}
        assert all(by_request[i] == s.output(i) for i in ids)        # every kept token was reported once
        return [s.output(i) for i in ids], [s.requests[i].finish_reason for i in ids], s.preemptions, s.steps

    free = run(False, (), 1024)
    assert [len(t) for t in free[0]] == limits
    # end tokens taken from what the requests do generate, so that some of them end early
    eos = (free[0][0][10], free[0][2][5], free[0][4][20])
    wait, ahead = run(False, eos, 1024), run(True, eos, 1024)
    assert ahead[:2] == wait[:2]
    assert "eos" in wait[1] and "length" in wait[1]
    assert any(len(t) < n for t, n in zip(wait[0], limits))
    # a pool so tight that running requests outgrow it and are preempted (and one of them with its
    # newest token still on its way)
    wait, ahead = run(False, (), 96), run(True, (), 96)
    assert ahead[:2] == wait[:2] and ahead[0] == free[0]
    assert wait[2] > 0 and ahead[2] > 0
    wait, ahead = run(False, eos[1:], 96), run(True, eos[1:], 96)
    assert ahead[:2] == wait[:2] and ahead[2] > 0
