"""Throughput measurements of the engine; `bench.py` at the repository's root and
`python -m litinfer_amd bench` both run `main` here.

    bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L] [--dtype bf16|fp32]
             [--mode headline|serving|long]

headline (default): the Qwen2-7B layer sizes.  A "step" is one decode step of the whole
batch through the engine's step function plus greedy sampling, the next tokens fed back on
the device (the host reads each step's tokens while the next step runs, as the scheduler
does with lookahead).  Beside this raw loop of steps the same batch sizes run through the
scheduler: 2,048-token prompts in portions, then 256 greedy tokens, with the time to the
first token and the time per token after it.  A prompt of 2,048 tokens is timed as one
step.  Every throughput stands beside its roofline: bytes a decode step has to read over
the HBM peak, flops of the prompt over the matrix peak of the dtype, and both also over
what a kernel that only reads, and one that only multiplies, reach on this GPU.

serving: the 1.5B layer sizes under continuous batching: 128 requests with prompts of 16
to 4,096 and outputs of 16 to 512 tokens arriving over time, half greedy, half at
temperature 0.7.  long: the 32B layer sizes with 8 prompts of 30,000 tokens in portions of
2,048, then 256 greedy tokens each.

Weights are random (drawn on the device), token ids are seeded synthetic ids.  In the raw
loop of steps the cache of every request is filled with random keys and values up to the
context length (their content does not change the work); the scheduler runs fill it by
computing the prompts.  One JSON line is printed; its shape follows the reference's own
harness where that has one (scripts/benchmark_cpu.py:133-141, 306-331: median/min/max of
repeats, time to first token, decode tokens a second, time per output token;
python/llaisys/models/qwen2.py:399-407).
"""
from __future__ import annotations

import argparse
import json
import statistics
import sys
import time
from typing import Dict, List, Optional

SHAPES = {
    "7b": {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_act": "silu",
           "num_hidden_layers": 28, "hidden_size": 3584, "num_attention_heads": 28, "num_key_value_heads": 4,
           "head_dim": 128, "intermediate_size": 18944, "vocab_size": 152064, "rope_theta": 1000000.0,
           "rms_norm_eps": 1e-6, "tie_word_embeddings": False, "use_sliding_window": False,
           "max_position_embeddings": 4096},
    "1.5b": {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_act": "silu",
             "num_hidden_layers": 28, "hidden_size": 1536, "num_attention_heads": 12, "num_key_value_heads": 2,
             "head_dim": 128, "intermediate_size": 8960, "vocab_size": 151936, "rope_theta": 10000.0,
             "rms_norm_eps": 1e-6, "tie_word_embeddings": False, "use_sliding_window": False,
             "max_position_embeddings": 8192},
    "32b": {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_act": "silu",
            "num_hidden_layers": 64, "hidden_size": 5120, "num_attention_heads": 40, "num_key_value_heads": 8,
            "head_dim": 128, "intermediate_size": 27648, "vocab_size": 152064, "rope_theta": 1000000.0,
            "rms_norm_eps": 1e-6, "tie_word_embeddings": False, "use_sliding_window": False,
            "max_position_embeddings": 32768},
    # further members of the family, for `--mode sweep --shape ...`
    "0.5b": {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_act": "silu",
             "num_hidden_layers": 24, "hidden_size": 896, "num_attention_heads": 14, "num_key_value_heads": 2,
             "head_dim": 64, "intermediate_size": 4864, "vocab_size": 151936, "rope_theta": 1000000.0,
             "rms_norm_eps": 1e-6, "tie_word_embeddings": True, "use_sliding_window": False,
             "max_position_embeddings": 32768},
    "3b": {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_act": "silu",
           "num_hidden_layers": 36, "hidden_size": 2048, "num_attention_heads": 16, "num_key_value_heads": 2,
           "head_dim": 128, "intermediate_size": 11008, "vocab_size": 151936, "rope_theta": 1000000.0,
           "rms_norm_eps": 1e-6, "tie_word_embeddings": True, "use_sliding_window": False,
           "max_position_embeddings": 32768},
    "14b": {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_act": "silu",
            "num_hidden_layers": 48, "hidden_size": 5120, "num_attention_heads": 40, "num_key_value_heads": 8,
            "head_dim": 128, "intermediate_size": 13824, "vocab_size": 152064, "rope_theta": 1000000.0,
            "rms_norm_eps": 1e-6, "tie_word_embeddings": False, "use_sliding_window": False,
            "max_position_embeddings": 32768},
    "72b": {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_act": "silu",
            "num_hidden_layers": 80, "hidden_size": 8192, "num_attention_heads": 64, "num_key_value_heads": 8,
            "head_dim": 128, "intermediate_size": 29568, "vocab_size": 152064, "rope_theta": 1000000.0,
            "rms_norm_eps": 1e-6, "tie_word_embeddings": False, "use_sliding_window": False,
            "max_position_embeddings": 32768},
}
QWEN2_7B = SHAPES["7b"]
CONTEXT = 4096
PREFILL_TOKENS = 2048
NEW_TOKENS = 256
PAGE = 16
HBM_PEAK = 8.0e12
FLOP_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}
ENGINE_DTYPE = {"bf16": "bfloat16", "fp32": "float32"}


def log(msg: str) -> None:
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


# ------------------------------------------------------------------ rooflines
def linear_params(c) -> int:
    h, nh, nkv, dh, inter = (c["hidden_size"], c["num_attention_heads"], c["num_key_value_heads"],
                             c["head_dim"], c["intermediate_size"])
    return (nh + 2 * nkv) * dh * h + h * nh * dh + 3 * h * inter


def kv_bytes_per_token(c, layers, es) -> int:
    return layers * 2 * c["num_key_value_heads"] * c["head_dim"] * es


def decode_bytes(c, layers, batch_ctx_tokens, es) -> float:
    """What a decode step has to read: every weight it uses once (matrices in the engine's
    dtype, the q/k/v biases in 32-bit), and the cache of the live requests."""
    w = layers * linear_params(c) * es
    w += layers * (c["num_attention_heads"] + 2 * c["num_key_value_heads"]) * c["head_dim"] * 4
    w += c["vocab_size"] * c["hidden_size"] * es
    return w + batch_ctx_tokens * kv_bytes_per_token(c, layers, es)


def prefill_flops(c, layers, t, start=0) -> float:
    """Flops of a portion of t tokens after `start` cached ones, logits for one row."""
    lin = 2.0 * t * layers * linear_params(c)
    keys = t * start + t * (t + 1) / 2.0                                  # causal: visible (query, key) pairs
    att = 4.0 * keys * c["num_attention_heads"] * c["head_dim"] * layers  # QK^T and PV
    return lin + att + 2.0 * c["vocab_size"] * c["hidden_size"]


def spread(values: List[float], scale: float = 1.0, digits: int = 3) -> Dict[str, float]:
    if not values:
        return {"median": None, "min": None, "max": None}
    return {"median": round(statistics.median(values) * scale, digits), "min": round(min(values) * scale, digits),
            "max": round(max(values) * scale, digits)}


def environment(dev) -> Dict[str, object]:
    """Where the numbers were measured (the reference's harness records the same kind of block:
    scripts/benchmark_cpu.py:306-325): the GPU, the versions of the runtime, of the driver and of
    torch, and the commit of this tree."""
    import os
    import platform
    import subprocess
    from pathlib import Path

    import torch
    env: Dict[str, object] = {"python": platform.python_version(), "torch": torch.__version__,
                              "hip": getattr(torch.version, "hip", None), "os": platform.platform(),
                              "command": sys.argv}
    try:
        p = torch.cuda.get_device_properties(dev)
        env.update(gpu=p.name, arch=getattr(p, "gcnArchName", None), compute_units=p.multi_processor_count,
                   memory_GiB=round(p.total_memory / 2 ** 30, 1),
                   max_clock_MHz=round(getattr(p, "clock_rate", 0) / 1000) or None,
                   memory_clock_MHz=round(getattr(p, "memory_clock_rate", 0) / 1000) or None)
    except Exception as e:                               # (no GPU: the block still says where it ran)
        env["gpu"] = f"unknown ({e})"
    for name, path in (("driver", "/sys/module/amdgpu/version"), ("driver_src", "/sys/module/amdgpu/srcversion"),
                       ("rocm", "/opt/rocm/.info/version")):
        try:
            env[name] = Path(path).read_text().strip()
        except OSError:
            env[name] = None
    root = Path(__file__).resolve().parent.parent
    try:
        env["git_commit"] = subprocess.run(["git", "-C", str(root), "rev-parse", "HEAD"], capture_output=True,
                                           text=True, timeout=10).stdout.strip() or None
        env["git_dirty"] = bool(subprocess.run(["git", "-C", str(root), "status", "--porcelain", "--untracked-files=no"],
                                               capture_output=True, text=True, timeout=10).stdout.strip())
    except (OSError, subprocess.SubprocessError):
        env["git_commit"] = None
    # the tree may be a copy without its history: a digest of the package's sources names it all the same
    import hashlib
    h = hashlib.sha256()
    pkg = Path(__file__).resolve().parent
    for f in sorted(list(pkg.rglob("*.py")) + list((pkg / "csrc").glob("*"))):
        if f.is_file():
            h.update(f.relative_to(pkg).as_posix().encode() + b"\0" + f.read_bytes())
    env["source_digest"] = h.hexdigest()[:16]
    env["omp_threads"] = os.environ.get("OMP_NUM_THREADS")
    return env


# ------------------------------------------------------- what the GPU reaches
def measure_reference(dev) -> Dict[str, float]:
    """A kernel that only reads (and one that copies) 2 GiB, a loop of bfloat16 MFMAs and a
    loop of float32 FMAs on registers: the rates the engine's kernels can be held against
    beside the published peaks."""
    import torch
    from .kernels import probe
    out = {}
    nbytes = 2 << 30
    src = torch.empty(nbytes, dtype=torch.uint8, device=dev).random_(0, 255)
    dst = torch.empty_like(src)

    def timed(fn, reps=5):
        fn()
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(reps):
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            fn()
            e.record()
            torch.cuda.synchronize()
            best = min(best, s.elapsed_time(e) * 1e-3)
        return best
    # the read rate depends on how the blocks walk through memory: one block a compute unit, each taking
    # 4 KB at a time with a stride of all blocks (a window of a few MB that moves through the buffer), reads
    # a fifth faster than sixteen blocks a unit; the best of the forms is the yardstick
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    out["read_GBps"] = round(max(nbytes / timed(lambda: probe.read(src, blocks=b)) for b in (cus, 2 * cus, 16 * cus)) / 1e9, 1)
    out["copy_GBps"] = round(2 * nbytes / timed(lambda: probe.copy(src, dst)) / 1e9, 1)      # read + written bytes
    del src, dst
    torch.cuda.empty_cache()
    blocks, iters = 256 * 8, 20000
    t = timed(lambda: probe.mfma(blocks, iters), reps=3)
    out["mfma_bf16_TFLOPs"] = round(probe.mfma_flops(blocks, iters) / t / 1e12, 1)
    t = timed(lambda: probe.fma(blocks * 4, iters), reps=3)
    out["fma_fp32_TFLOPs"] = round(probe.fma_flops(blocks * 4, iters) / t / 1e12, 1)
    return out


# ------------------------------------------------------------ the raw step loop
class StepLoop:
    """Decode steps of a fixed batch driven by hand: engine.step + greedy sampling, tokens
    fed back on the device."""

    def __init__(self, eng, cfg, sampler, rng):
        self.eng, self.cfg, self.sampler, self.rng = eng, cfg, sampler, rng

    def run(self, batch: int, steps: int, warmup: int, context: int):
        import torch
        from .engine import StepEntry
        from .sampling import SamplingParams
        eng = self.eng
        start_ctx = context - steps - warmup - 1          # one more step fits afterwards: the check against an eager step
        rids = [f"d{batch}_{i}" for i in range(batch)]
        for r in rids:                               # the cache "holds" start_ctx tokens of each request
            eng.cache.admit(r)
            eng.cache.reserve(r, start_ctx)
            eng.cache.commit(r, start_ctx)
        toks = self.rng.integers(0, self.cfg["vocab_size"], batch).tolist()
        params, counters = [SamplingParams()] * batch, [0] * batch
        state = {"pending": None, "n": 0, "logits": None}

        def one():
            first = state["n"] == 0
            logits = eng.step([StepEntry(r, [t], [0], None if first else [i])
                               for i, (r, t) in enumerate(zip(rids, toks))])
            handle = self.sampler.sample_async(logits, params, counters, out=eng.feedback)
            if state["pending"] is not None:
                state["pending"].result()
            state["pending"], state["n"], state["logits"] = handle, state["n"] + 1, logits
        for _ in range(warmup):
            one()
        if state["pending"] is not None:
            state["pending"].result()
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(steps):
            one()
        last = state["pending"].result()             # the last step's tokens have reached the host
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        # outside the timed region: what was computed is finite, and a recorded step gives the tokens
        # of an eager step of the same batch
        logits = state["logits"]
        if not bool(torch.isfinite(logits).all()):
            raise RuntimeError(f"bench: non-finite logits in the decode loop at batch {batch}")
        self._check_against_eager(rids, last, batch)
        ctx_tokens = batch * (start_ctx + warmup + steps / 2.0)
        for r in rids:
            eng.finish(r)
        return dt, ctx_tokens

    def _check_against_eager(self, rids, last_tokens, batch):
        """One more step of the same requests twice: as the engine runs it (recorded, if it
        records) and eagerly from a copy of the cache's state; the greedy tokens must agree."""
        import torch
        from .engine import StepEntry
        from .sampling import SamplingParams
        eng = self.eng
        entries = [StepEntry(r, [int(t)], [0]) for r, t in zip(rids, last_tokens)]
        a = eng.step(entries).clone()
        was = eng.use_graphs
        # the same positions again: pretend the step has not happened (lengths only; the pages stay)
        for r in rids:
            eng.cache.rewind(r, 1)
        eng.use_graphs = False
        try:
            b = eng.step(entries).clone()
        finally:
            eng.use_graphs = was
        # The two runs may cut the keys of the decode attention differently (a recorded step is laid
        # out for the block table's padded width), so they agree to rounding, not to the bit: the
        # logits must be close, and where the greedy tokens differ the two candidates must be that close.
        params = [SamplingParams()] * batch
        ta = self.sampler.sample(a, params, [0] * batch)
        tb = self.sampler.sample(b, params, [0] * batch)
        worst = float((a - b).abs().max())
        scale = float(a.abs().max())
        tol = (3e-2 if self.eng.rt.dtype is torch.bfloat16 else 1e-4) * scale
        if not worst <= tol:
            raise RuntimeError(f"bench: a recorded decode step and an eager one of the same batch of {batch} differ by "
                               f"{worst:.3e} in a logit (largest logit {scale:.3e})")
        for i, (x, y) in enumerate(zip(ta, tb)):
            if x != y and float(a[i, x] - a[i, y]) > 2 * worst:
                raise RuntimeError(f"bench: a recorded decode step and an eager one of the same batch of {batch} "
                                   f"chose different tokens for row {i} (logits {float(a[i, x]):.4f} and {float(a[i, y]):.4f}, "
                                   f"largest logit difference {worst:.3e})")


# ------------------------------------------------------ through the scheduler
def run_scheduler(eng, cfg, requests, *, max_batch_tokens: int, chunk_size: int, arrivals=None,
                  what: str = "") -> Dict[str, object]:
    """Submit the requests (each: prompt, new tokens, sampling) to the scheduler, at their
    arrival times if given (seconds from the start) or all at once, and run it dry.
    Returns wall tokens a second and the distributions the reference's harness reports."""
    import torch
    from .engine import Scheduler
    sched = Scheduler(eng, max_batch_tokens=max_batch_tokens, chunk_size=chunk_size, lookahead=True)
    order = sorted(range(len(requests)), key=lambda i: arrivals[i] if arrivals else 0.0)
    submitted, first_at, last_at, count = {}, {}, {}, {}
    step_log = []                                    # (time after the step, tokens it produced)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    nxt = 0
    busy_steps = 0
    next_note = t0 + 20.0
    while nxt < len(order) or sched.has_unfinished():
        now = time.perf_counter() - t0
        while nxt < len(order) and (not arrivals or arrivals[order[nxt]] <= now):
            i = order[nxt]
            prompt, new, params = requests[i]
            rid = sched.add_request(prompt, new, params, rid=i)
            submitted[rid] = arrivals[i] if arrivals else now
            nxt += 1
        if not sched.has_unfinished():
            time.sleep(max(0.0, min(0.002, arrivals[order[nxt]] - now)))     # nothing to do until the next arrival
            continue
        produced = sched.step()
        busy_steps += 1
        now = time.perf_counter() - t0
        for rid, _ in produced:
            first_at.setdefault(rid, now)
            last_at[rid] = now
            count[rid] = count.get(rid, 0) + 1
        step_log.append((now, len(produced)))
        if time.perf_counter() > next_note:
            log(f"{what}: {now:.0f} s, {sum(count.values())} tokens, {len(sched.running)} running, "
                f"{len(sched.waiting)} waiting")
            next_note = time.perf_counter() + 20.0
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    reasons = {}
    for r in sched.requests.values():
        reasons[r.finish_reason] = reasons.get(r.finish_reason, 0) + 1
    generated = sum(len(r.generated) for r in sched.requests.values())
    prompt_tokens = sum(len(p) for p, _, _ in requests)
    ttft = [first_at[r] - submitted[r] for r in first_at]
    tpot = [(last_at[r] - first_at[r]) / (count[r] - 1) for r in first_at if count[r] > 1]
    eng.cache.check_invariants()
    # the stretch in which every request decodes: from the last request's first token to the first request's end
    lo, hi = max(first_at.values()), min(last_at.values())
    phase = [(t, n) for t, n in step_log if lo < t <= hi]
    decode_phase = None
    if len(phase) >= 8:
        span = phase[-1][0] - lo
        decode_phase = {"steps": len(phase), "tok_s": round(sum(n for _, n in phase) / span, 1),
                        "ms_per_step": round(span / len(phase) * 1e3, 4)}
    return {"requests": len(requests), "prompt_tokens": prompt_tokens, "generated_tokens": generated,
            "decode_phase": decode_phase,
            "wall_s": round(wall, 3), "tok_s": round(generated / wall, 1),
            "total_tok_s": round((generated + prompt_tokens) / wall, 1),
            "ttft_ms": spread(ttft, 1e3), "tpot_ms": spread(tpot, 1e3), "steps": busy_steps,
            "preemptions": sched.preemptions, "finished": reasons}


# -------------------------------------------------------------------- modes
def headline(a) -> Dict[str, object]:
    import numpy as np
    import torch
    from .engine import Engine, StepEntry
    from .sampling import Sampler, SamplingParams

    cfg = dict(QWEN2_7B, num_hidden_layers=a.layers)
    es = 2 if a.dtype == "bf16" else 4
    dev = "cuda:0"
    max_b = max(a.batch, 1 if a.no_points else 64)
    ref = None if a.no_reference else measure_reference(dev)
    if ref:
        log(f"this GPU: read {ref['read_GBps']} GB/s, copy {ref['copy_GBps']} GB/s, "
            f"bf16 MFMA loop {ref['mfma_bf16_TFLOPs']} TFLOP/s, fp32 FMA loop {ref['fma_fp32_TFLOPs']} TFLOP/s")
    t0 = time.time()
    eng = Engine.from_random(cfg, seed=0, dtype=ENGINE_DTYPE[a.dtype], device=dev, page_size=PAGE,
                             num_pages=max_b * CONTEXT // PAGE + PREFILL_TOKENS // PAGE, max_seqs=max_b + 1,
                             page_order_seed=None if a.page_order_seed < 0 else a.page_order_seed)
    for g in eng.cache.groups:                       # synthetic cache content
        for data in g.data.values():
            flat = data.view(-1)
            for i in range(0, flat.numel(), 1 << 28):
                flat[i:i + (1 << 28)].normal_(0, 0.5)
    torch.cuda.synchronize()
    log(f"model and cache ready in {time.time() - t0:.1f} s ({eng.model.weight_bytes() / 1e9:.2f} GB of weights)")
    sampler = Sampler(dev)
    rng = np.random.default_rng(0)
    loop = StepLoop(eng, cfg, sampler, rng)

    def frac_of(nbytes, seconds):
        return round(nbytes / seconds / HBM_PEAK, 4)

    dt, ctx_tokens = loop.run(a.batch, a.steps, a.warmup, CONTEXT)
    # the headline is that first timing of exactly `steps` steps; it is repeated (each repeat: its own
    # requests, warm-up and `steps` timed steps) for the spread
    decode_ms = [dt / a.steps * 1e3]
    for _ in range(max(0, a.repeats - 1)):
        d, _ = loop.run(a.batch, a.steps, a.warmup, CONTEXT)
        decode_ms.append(d / a.steps * 1e3)
    ms = dt / a.steps * 1e3
    value = a.batch * a.steps / dt
    nbytes = decode_bytes(cfg, a.layers, ctx_tokens, es)
    out = {
        "metric": f"decode tok/s (Qwen2-7B shape, batch {a.batch}, context {CONTEXT})", "value": round(value, 2),
        "unit": "tok/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": a.dtype,
        "data": "synthetic: seeded random token ids, random weights N(0, 0.02), random cache content in the loop of steps, "
                + ("pages handed out in the order of their numbers" if a.page_order_seed < 0 else "pages handed out in a shuffled order"),
        "config": {"model": "Qwen2-7B shape", "num_hidden_layers": a.layers,
                   "full_num_hidden_layers": QWEN2_7B["num_hidden_layers"], "hidden_size": cfg["hidden_size"],
                   "num_attention_heads": cfg["num_attention_heads"],
                   "num_key_value_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
                   "intermediate_size": cfg["intermediate_size"], "vocab_size": cfg["vocab_size"],
                   "global_batch": a.batch, "seq_len": CONTEXT, "context_len": CONTEXT,
                   "prefill_tokens": PREFILL_TOKENS, "page_size": PAGE, "rope_theta": cfg["rope_theta"],
                   "rms_norm_eps": cfg["rms_norm_eps"], "tie_word_embeddings": False,
                   "parallelism": "none (1 GPU)"},
        "roofline": {"bound": "hbm", "achieved": round(nbytes / (ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK / 1e9,
                     "unit": "GB/s", "frac": frac_of(nbytes, ms * 1e-3)},
    }
    out["repeats"] = {"n": len(decode_ms), "decode_ms_per_step": spread(decode_ms, 1.0, 4)}
    if ref:
        out["roofline"]["frac_of_measured_read"] = round(nbytes / (ms * 1e-3) / (ref["read_GBps"] * 1e9), 4)
    if not a.no_prefill:
        prompt = rng.integers(0, cfg["vocab_size"], PREFILL_TOKENS).tolist()
        times = []
        for i in range(1 + (max(a.repeats, 4) if a.dtype == "bf16" else max(a.repeats, 2))):   # one to warm up, the best of the rest
            torch.cuda.synchronize()
            t = time.perf_counter()
            logits = eng.step([StepEntry(f"p{i}", prompt, [PREFILL_TOKENS - 1])])
            sampler.sample(logits, [SamplingParams()], [0])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t)
            if not bool(torch.isfinite(logits).all()):
                raise RuntimeError("bench: non-finite logits after the prompt")
            eng.finish(f"p{i}")
        pt = min(times[1:])
        flops = prefill_flops(cfg, a.layers, PREFILL_TOKENS)
        out["prefill"] = {"value": round(PREFILL_TOKENS / pt, 1), "tokens": PREFILL_TOKENS,
                          "ms": round(pt * 1e3, 3), "frac": round(flops / pt / FLOP_PEAK[a.dtype], 4)}
        out["repeats"]["prefill_ms"] = spread(times[1:], 1e3, 3)
        if ref:
            measured = ref["mfma_bf16_TFLOPs"] if a.dtype == "bf16" else ref["fma_fp32_TFLOPs"]
            out["prefill"]["frac_of_measured_loop"] = round(flops / pt / (measured * 1e12), 4)
    if not a.no_points:
        pts, fracs = {}, {}
        for b in (1, 64):
            n = max(8, a.steps // 2)
            d, ctx_b = loop.run(b, n, 4, CONTEXT)
            pts[f"decode_b{b}"] = round(b * n / d, 2)
            fracs[f"decode_b{b}"] = frac_of(decode_bytes(cfg, a.layers, ctx_b, es), d / n)
        out["points"] = pts
        out["points_frac"] = fracs
    if ref:
        out["reference"] = ref
    if not a.no_scheduler:
        # the headline workload through the scheduler: prompts of 2,048 tokens, then 256 greedy tokens
        sch = {}
        # (in 32-bit the prompts of 64 requests alone take half a minute: the batch and one request there)
        for b in ((a.batch,) if a.no_points else (a.batch, 64, 1) if a.dtype == "bf16" else (a.batch, 1)):
            reqs = [(rng.integers(0, cfg["vocab_size"], PREFILL_TOKENS).tolist(), NEW_TOKENS, SamplingParams())
                    for _ in range(b)]
            r = run_scheduler(eng, cfg, reqs, max_batch_tokens=PREFILL_TOKENS + 64, chunk_size=PREFILL_TOKENS,
                              what=f"scheduler, {b} requests")
            tpot = r["tpot_ms"]["median"]
            ph = r["decode_phase"]
            if ph:                                   # all b requests decode: contexts of 2,048 + what has been generated
                mean_ctx = b * (PREFILL_TOKENS + NEW_TOKENS / 2.0)
                ph["frac"] = frac_of(decode_bytes(cfg, a.layers, mean_ctx, es), ph["ms_per_step"] * 1e-3)
            sch[f"b{b}"] = r
            log(f"scheduler, {b} requests: {r['tok_s']} generated tok/s over all, TTFT median {r['ttft_ms']['median']} ms, "
                f"TPOT median {tpot} ms; while all decode: {ph}")
        out["scheduler"] = sch
    out["environment"] = environment(dev)
    if not a.no_points and not a.no_small:
        # the reference's own benchmark model (DeepSeek-R1-Distill-Qwen-1.5B layer sizes), same run: decode at
        # 1, 8 and 64 requests, context 4,096, each with its fraction of the HBM peak
        del loop, eng
        torch.cuda.empty_cache()
        out["points_1p5b"] = small_points(a, dev, sampler, rng)
    return out


def small_points(a, dev, sampler, rng) -> Dict[str, object]:
    import torch
    from .engine import Engine
    cfg = dict(SHAPES["1.5b"])
    layers = cfg["num_hidden_layers"]
    es = 2 if a.dtype == "bf16" else 4
    t0 = time.time()
    eng = Engine.from_random(cfg, seed=0, dtype=ENGINE_DTYPE[a.dtype], device=dev, page_size=PAGE,
                             num_pages=64 * CONTEXT // PAGE + 64, max_seqs=65,
                             page_order_seed=None if a.page_order_seed < 0 else a.page_order_seed)
    for g in eng.cache.groups:
        for data in g.data.values():
            data.view(-1).normal_(0, 0.5)
    loop = StepLoop(eng, cfg, sampler, rng)
    pts: Dict[str, object] = {"model": "DeepSeek-R1-Distill-Qwen-1.5B shape", "num_hidden_layers": layers, "context_len": CONTEXT}
    for b in (1, 8, 64):
        n = max(8, a.steps // 2) if b != 8 else a.steps
        d, ctx_b = loop.run(b, n, 4, CONTEXT)
        pts[f"decode_b{b}"] = {"tok_s": round(b * n / d, 1), "ms_per_step": round(d / n * 1e3, 4),
                               "frac": round(decode_bytes(cfg, layers, ctx_b, es) / (d / n) / HBM_PEAK, 4)}
    torch.cuda.synchronize()
    log(f"1.5B shape in {time.time() - t0:.1f} s: {pts}")
    return pts


def sweep(a) -> Dict[str, object]:
    """Decode steps and prompts at further sizes of the 7B layer shape: contexts of 1,024 to 16,384
    tokens at 1, 8 and 64 requests, prompts of 512 to 8,192 tokens and a portion of 1,024 tokens
    behind 15,360 cached ones; each with its fraction of the published peak."""
    import numpy as np
    import torch
    from .engine import Engine, StepEntry
    from .sampling import Sampler, SamplingParams

    cfg = dict(SHAPES[a.shape], num_hidden_layers=a.layers, max_position_embeddings=32768)
    es = 2 if a.dtype == "bf16" else 4
    dev = "cuda:0"
    contexts, batches = ((1024, 4096, 16384) if a.shape == "7b" else (4096,)), (1, 8, 64)
    eng = Engine.from_random(cfg, seed=0, dtype=ENGINE_DTYPE[a.dtype], device=dev, page_size=PAGE,
                             num_pages=max(batches) * max(contexts) // PAGE + 1024, max_seqs=max(batches) + 1)
    for g in eng.cache.groups:
        for data in g.data.values():
            flat = data.view(-1)
            for i in range(0, flat.numel(), 1 << 28):
                flat[i:i + (1 << 28)].normal_(0, 0.5)
    sampler = Sampler(dev)
    rng = np.random.default_rng(0)
    loop = StepLoop(eng, cfg, sampler, rng)
    decode = {}
    for ctx in contexts:
        for b in batches:
            dt, ctx_tokens = loop.run(b, a.steps, a.warmup, ctx)
            nbytes = decode_bytes(cfg, a.layers, ctx_tokens, es)
            decode[f"ctx{ctx}_b{b}"] = {"tok_s": round(b * a.steps / dt, 1), "ms_per_step": round(dt / a.steps * 1e3, 3),
                                        "frac": round(nbytes / dt * a.steps / HBM_PEAK, 4)}
            log(f"decode, context {ctx}, batch {b}: {decode[f'ctx{ctx}_b{b}']}")
    prefill = {}
    for tokens, start in (((512, 0), (2048, 0), (8192, 0), (1024, 15360)) if a.shape == "7b" else ((2048, 0),)):
        ids = rng.integers(0, cfg["vocab_size"], start + tokens).tolist()
        times = []
        for i in range(4):
            rid = f"s{tokens}_{start}_{i}"
            if start:                                   # the cached part first, in portions; not timed
                for o in range(0, start, 2048):
                    eng.step([StepEntry(rid, ids[o:o + 2048], [])])
            torch.cuda.synchronize()
            t = time.perf_counter()
            logits = eng.step([StepEntry(rid, ids[start:], [tokens - 1])])
            sampler.sample(logits, [SamplingParams()], [0])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t)
            eng.finish(rid)
        pt = min(times[1:])
        flops = prefill_flops(cfg, a.layers, tokens, start)
        key = f"t{tokens}" + (f"_after{start}" if start else "")
        prefill[key] = {"tok_s": round(tokens / pt, 1), "ms": round(pt * 1e3, 3), "frac": round(flops / pt / FLOP_PEAK[a.dtype], 4)}
        log(f"prompt of {tokens} tokens behind {start}: {prefill[key]}")
    best = decode["ctx4096_b8"]
    return {"metric": f"decode tok/s and prompt tok/s at further sizes (Qwen2 {a.shape} shape)", "value": best["tok_s"], "unit": "tok/s",
            "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": best["ms_per_step"], "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": a.dtype, "data": "synthetic: seeded random token ids, random weights, random cache content",
            "config": {"model": f"Qwen2 {a.shape} shape", "num_hidden_layers": a.layers, "full_num_hidden_layers": SHAPES[a.shape]["num_hidden_layers"],
                       "page_size": PAGE, "parallelism": "none (1 GPU)"},
            "decode": decode, "prefill_at": prefill}


def serving(a) -> Dict[str, object]:
    """Continuous batching at the 1.5B layer sizes: 128 requests of random lengths arriving over time, half of them sampled."""
    import numpy as np
    import torch
    from .engine import Engine
    from .sampling import SamplingParams
    cfg = dict(SHAPES["1.5b"])
    if a.layers:
        cfg["num_hidden_layers"] = a.layers
    layers = cfg["num_hidden_layers"]
    es = 2 if a.dtype == "bf16" else 4
    rng = np.random.default_rng(1)
    n = a.requests
    plen = rng.integers(16, 4097, n)
    olen = rng.integers(16, 513, n)
    arrivals = np.cumsum(rng.exponential(1.0 / a.arrival_rate, n)).tolist()
    reqs = []
    for i in range(n):
        params = SamplingParams() if i % 2 == 0 else SamplingParams(temperature=0.7, seed=i)
        reqs.append((rng.integers(0, cfg["vocab_size"], int(plen[i])).tolist(), int(olen[i]), params))
    pool_tokens = a.pool_tokens or int(sum(-(-int(p + o) // PAGE) * PAGE for p, o in zip(plen, olen)))
    eng = Engine.from_random(cfg, seed=0, dtype=ENGINE_DTYPE[a.dtype], device="cuda:0", page_size=PAGE,
                             num_pages=pool_tokens // PAGE, max_seqs=a.max_seqs)
    torch.cuda.synchronize()
    log(f"serving: {n} requests, {int(plen.sum())} prompt and {int(olen.sum())} output tokens, "
        f"pool of {pool_tokens} tokens, {a.max_seqs} slots")
    warm = [(rng.integers(0, cfg["vocab_size"], 512).tolist(), 8, SamplingParams()) for _ in range(4)]
    run_scheduler(eng, cfg, warm, max_batch_tokens=a.max_batch_tokens, chunk_size=a.chunk_size, what="warm-up")
    r = run_scheduler(eng, cfg, reqs, max_batch_tokens=a.max_batch_tokens, chunk_size=a.chunk_size,
                      arrivals=arrivals, what="serving")
    return {
        "metric": "generated tok/s under continuous batching (DeepSeek-R1-Distill-Qwen-1.5B shape, 128 requests)",
        "value": r["tok_s"], "unit": "tok/s", "n_gpus": 1, "steps": r["steps"], "warmup": 0,
        "ms_per_step": round(r["wall_s"] / max(1, r["steps"]) * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": a.dtype,
        "data": "synthetic: seeded random token ids, prompt lengths U[16,4096], output lengths U[16,512], "
                "exponential arrivals, half greedy and half at temperature 0.7, random weights",
        "config": {"model": "DeepSeek-R1-Distill-Qwen-1.5B shape", "num_hidden_layers": layers,
                   "full_num_hidden_layers": SHAPES["1.5b"]["num_hidden_layers"], "hidden_size": cfg["hidden_size"],
                   "num_attention_heads": cfg["num_attention_heads"], "num_key_value_heads": cfg["num_key_value_heads"],
                   "head_dim": cfg["head_dim"], "intermediate_size": cfg["intermediate_size"],
                   "vocab_size": cfg["vocab_size"], "global_batch": a.max_seqs, "seq_len": cfg["max_position_embeddings"],
                   "requests": n, "arrival_rate_per_s": a.arrival_rate, "pool_tokens": pool_tokens,
                   "max_batch_tokens": a.max_batch_tokens, "chunk_size": a.chunk_size, "page_size": PAGE,
                   "parallelism": "none (1 GPU)"},
        "serving": r,
        "bytes_per_cached_token": kv_bytes_per_token(cfg, layers, es),
    }


def long_prompts(a) -> Dict[str, object]:
    """Long prompts at the 32B layer sizes: 8 prompts of 30,000 tokens in portions, then 256 greedy tokens each."""
    import numpy as np
    import torch
    from .engine import Engine
    from .sampling import SamplingParams
    cfg = dict(SHAPES["32b"])
    if a.layers:
        cfg["num_hidden_layers"] = a.layers
    layers = cfg["num_hidden_layers"]
    es = 2 if a.dtype == "bf16" else 4
    rng = np.random.default_rng(2)
    n, plen, new, chunk = a.requests or 8, a.prompt_len, NEW_TOKENS, 2048
    per_req = -(-(plen + new) // PAGE) * PAGE
    t0 = time.time()
    eng = Engine.from_random(cfg, seed=0, dtype=ENGINE_DTYPE[a.dtype], device="cuda:0", page_size=PAGE,
                             num_pages=n * per_req // PAGE, max_seqs=n)
    torch.cuda.synchronize()
    log(f"long: model ready in {time.time() - t0:.0f} s, {eng.model.weight_bytes() / 1e9:.1f} GB of weights, "
        f"{n * per_req * kv_bytes_per_token(cfg, layers, es) / 1e9:.1f} GB of pages")
    reqs = [(rng.integers(0, cfg["vocab_size"], plen).tolist(), new, SamplingParams()) for _ in range(n)]
    warm = [(rng.integers(0, cfg["vocab_size"], 3000).tolist(), 4, SamplingParams())]
    run_scheduler(eng, cfg, warm, max_batch_tokens=chunk + n, chunk_size=chunk, what="warm-up")
    r = run_scheduler(eng, cfg, reqs, max_batch_tokens=chunk + n, chunk_size=chunk, what="long")
    checked = check_long_decode(eng, cfg, reqs[0][0], chunk)
    # the prompts run one after the other in portions; the last request's first token marks their end
    prefill_s = r["ttft_ms"]["max"] * 1e-3
    flops = sum(prefill_flops(cfg, layers, min(chunk, plen - s), s) - 2.0 * cfg["vocab_size"] * cfg["hidden_size"]
                for s in range(0, plen, chunk)) * n
    # the decode step is timed where all requests decode (a request's time per token also holds the
    # portions of the prompts that were computed between its tokens)
    ph = r["decode_phase"] or {"ms_per_step": r["tpot_ms"]["median"], "steps": 0}
    tpot = ph["ms_per_step"]
    mean_ctx = n * (plen + new / 2.0)
    return {
        "metric": f"decode tok/s after {n} prompts of {plen} tokens (Qwen2.5-32B shape)",
        "value": round(n / (tpot * 1e-3), 2), "unit": "tok/s", "n_gpus": 1, "steps": ph["steps"], "warmup": 0,
        "ms_per_step": tpot, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": a.dtype,
        "data": "synthetic: seeded random token ids, random weights",
        "config": {"model": "Qwen2.5-32B shape", "num_hidden_layers": layers,
                   "full_num_hidden_layers": SHAPES["32b"]["num_hidden_layers"], "hidden_size": cfg["hidden_size"],
                   "num_attention_heads": cfg["num_attention_heads"], "num_key_value_heads": cfg["num_key_value_heads"],
                   "head_dim": cfg["head_dim"], "intermediate_size": cfg["intermediate_size"],
                   "vocab_size": cfg["vocab_size"], "global_batch": n, "seq_len": cfg["max_position_embeddings"],
                   "prompt_tokens": plen, "new_tokens": new, "chunk_size": chunk, "page_size": PAGE,
                   "parallelism": "none (1 GPU)"},
        "roofline": {"bound": "hbm", "achieved": round(decode_bytes(cfg, layers, mean_ctx, es) / (tpot * 1e-3) / 1e9, 1),
                     "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(decode_bytes(cfg, layers, mean_ctx, es) / (tpot * 1e-3) / HBM_PEAK, 4)},
        "prefill": {"value": round(n * plen / prefill_s, 1), "tokens": n * plen, "ms": round(prefill_s * 1e3, 1),
                    "frac": round(flops / prefill_s / FLOP_PEAK[a.dtype], 4)},
        "scheduler": r,
        "decode_row_checked": checked,
    }


def check_long_decode(eng, cfg, prompt, chunk) -> Dict[str, object]:
    """One request's prompt once more through the step function in portions, a few tokens decoded until
    its step is a recorded one, and then one decoded row twice: as the engine runs it (replayed) and
    eagerly.  The logits must agree to rounding (the reference's own regression at its longest lengths
    compares tokens, test/test_kv_cache.py:52-66)."""
    import numpy as np
    import torch
    from .engine import StepEntry
    from .sampling import Sampler
    t0 = time.time()
    rid = "long_check"
    logits = None
    for o in range(0, len(prompt), chunk):
        part = prompt[o:o + chunk]
        logits = eng.step([StepEntry(rid, part, [len(part) - 1] if o + chunk >= len(prompt) else [])])
    sampler = Sampler(eng.rt.device)
    loop = StepLoop(eng, cfg, sampler, np.random.default_rng(3))
    tok = int(torch.argmax(logits[0]))
    replays = eng.graph_replays
    for _ in range(eng.graph_after + 1):
        logits = eng.step([StepEntry(rid, [tok], [0])])
        tok = int(torch.argmax(logits[0]))
    recorded = eng.graph_replays > replays
    loop._check_against_eager([rid], [tok], 1)
    eng.finish(rid)
    out = {"context": len(prompt) + eng.graph_after + 2, "recorded_step": recorded, "seconds": round(time.time() - t0, 1)}
    log(f"long: a decoded row behind {out['context']} keys, recorded against eager: equal to rounding ({out})")
    return out


def main(argv: Optional[List[str]] = None) -> int:
    ap = argparse.ArgumentParser(prog="bench.py", description=__doc__.split("\n\n")[0])
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has (named in `config`)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--mode", default="headline", choices=["headline", "serving", "long", "sweep"])
    ap.add_argument("--shape", default="7b", choices=sorted(SHAPES), help="sweep: the member of the family whose layer sizes are taken")
    ap.add_argument("--page-order-seed", type=int, default=0,
                    help="headline: the cache's pages are handed out in a shuffled order, as a pool that has served requests "
                         "does (negative: in the order of their numbers; a request's keys then lie in one piece, and "
                         "how the pieces of a batch fall onto the memory's channels moves a batch-64 step by 7 %%)")
    ap.add_argument("--no-points", action="store_true", help="headline: skip the batch 1 and 64 points")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-scheduler", action="store_true", help="headline: skip the runs through the scheduler")
    ap.add_argument("--no-reference", action="store_true", help="headline: skip the measured read / MFMA rates")
    ap.add_argument("--no-small", action="store_true", help="headline: skip the decode points at the 1.5B layer sizes")
    ap.add_argument("--repeats", type=int, default=3, help="headline: timings of `steps` decode steps and of the prompt (median/min/max)")
    ap.add_argument("--requests", type=int, default=None, help="serving: number of requests (128); long: 8")
    ap.add_argument("--arrival-rate", type=float, default=32.0, help="serving: requests a second")
    ap.add_argument("--pool-tokens", type=int, default=None, help="serving: tokens the cache pool holds (default: all)")
    ap.add_argument("--max-seqs", type=int, default=128, help="serving: requests that may run at a time")
    ap.add_argument("--max-batch-tokens", type=int, default=2048)
    ap.add_argument("--chunk-size", type=int, default=1024)
    ap.add_argument("--prompt-len", type=int, default=30000, help="long: tokens of each prompt")
    a = ap.parse_args(argv)
    if a.gpus != 1:
        print(f"bench.py: this engine runs on ONE GPU; --gpus {a.gpus} is not supported", flush=True)
        return 2
    if a.mode == "headline":
        a.layers = a.layers or QWEN2_7B["num_hidden_layers"]
        out = headline(a)
    elif a.mode == "sweep":
        a.layers = a.layers or SHAPES[a.shape]["num_hidden_layers"]
        a.steps, a.warmup = min(a.steps, 32), min(a.warmup, 4)
        out = sweep(a)
    elif a.mode == "serving":
        a.requests = a.requests or 128
        out = serving(a)
    else:
        out = long_prompts(a)
    if "environment" not in out:
        out["environment"] = environment("cuda:0")
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
