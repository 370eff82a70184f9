#!/usr/bin/env python3
"""Decode and prefill throughput of the engine at the Qwen2-7B layer sizes.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L]

A "step" is one decode step of the whole batch through the engine's step
function plus greedy sampling, the next tokens fed back (on the device: the
host reads each step's tokens while the next step runs, as the scheduler does
with lookahead).  Weights are random
(drawn on the device), token ids are seeded synthetic ids, and the cache of
every request is filled with random keys and values up to the context length
before the timed steps (their content does not change the work).  One JSON
line is printed.
"""
from __future__ import annotations

import argparse
import json
import sys
import time

QWEN2_7B = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_act": "silu",
    "num_hidden_layers": 28, "hidden_size": 3584, "num_attention_heads": 28, "num_key_value_heads": 4,
    "head_dim": 128, "intermediate_size": 18944, "vocab_size": 152064, "rope_theta": 1000000.0,
    "rms_norm_eps": 1e-6, "tie_word_embeddings": False, "use_sliding_window": False,
    "max_position_embeddings": 4096,
}
CONTEXT = 4096
PREFILL_TOKENS = 2048
PAGE = 16
HBM_PEAK = 8.0e12
FLOP_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}


def linear_params(c) -> int:
    h, nh, nkv, dh, inter = (c["hidden_size"], c["num_attention_heads"], c["num_key_value_heads"],
                             c["head_dim"], c["intermediate_size"])
    return (nh + 2 * nkv) * dh * h + h * nh * dh + 3 * h * inter


def decode_bytes(c, layers, batch_ctx_tokens, es) -> float:
    """What a decode step has to read: every weight it uses once, and the cache
    of the live requests."""
    w = layers * (linear_params(c) + (c["num_attention_heads"] + 2 * c["num_key_value_heads"]) * c["head_dim"] / es * 4)
    w += c["vocab_size"] * c["hidden_size"]
    kv = batch_ctx_tokens * layers * 2 * c["num_key_value_heads"] * c["head_dim"]
    return (w + kv) * es


def prefill_flops(c, layers, t) -> float:
    lin = 2.0 * t * layers * linear_params(c)
    att = 2.0 * t * t * c["num_attention_heads"] * c["head_dim"] * layers      # causal: QK^T and PV over half
    return lin + att + 2.0 * c["vocab_size"] * c["hidden_size"]


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=QWEN2_7B["num_hidden_layers"])
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 points")
    ap.add_argument("--no-prefill", action="store_true")
    a = ap.parse_args()
    if a.gpus != 1:
        print(f"bench.py: this engine runs on ONE GPU; --gpus {a.gpus} is not supported", flush=True)
        return 2

    import numpy as np
    import torch
    from litinfer_amd.engine import Engine, StepEntry
    from litinfer_amd.sampling import Sampler, SamplingParams

    cfg = dict(QWEN2_7B, num_hidden_layers=a.layers)
    es = 2 if a.dtype == "bf16" else 4
    dev = "cuda:0"
    max_b = max(a.batch, 1 if a.no_points else 64)
    t0 = time.time()
    eng = Engine.from_random(cfg, seed=0, dtype={"bf16": "bfloat16", "fp32": "float32"}[a.dtype], device=dev,
                             page_size=PAGE, num_pages=max_b * CONTEXT // PAGE + PREFILL_TOKENS // PAGE,
                             max_seqs=max_b + 1)
    for g in eng.cache.groups:                       # synthetic cache content
        flat = g.data.view(-1)
        for i in range(0, flat.numel(), 1 << 28):
            flat[i:i + (1 << 28)].normal_(0, 0.5)
    torch.cuda.synchronize()
    print(f"[bench] model and cache ready in {time.time() - t0:.1f} s "
          f"({eng.model.weight_bytes() / 1e9:.2f} GB of weights)", file=sys.stderr, flush=True)
    sampler = Sampler(dev)
    rng = np.random.default_rng(0)

    def decode_run(batch: int, steps: int, warmup: int):
        start_ctx = CONTEXT - steps - warmup
        rids = [f"d{batch}_{i}" for i in range(batch)]
        for r in rids:                               # the cache "holds" start_ctx tokens of each request
            eng.cache.admit(r)
            eng.cache.reserve(r, start_ctx)
            eng.cache.commit(r, start_ctx)
        toks = rng.integers(0, cfg["vocab_size"], batch).tolist()
        params, counters = [SamplingParams()] * batch, [0] * batch
        state = {"pending": None, "n": 0}

        def one():
            # as the scheduler does with lookahead: the sampled ids stay on the device and the
            # next step takes them from the engine's feedback buffer; the host reads them one
            # step later, while the device is at work on the next step
            first = state["n"] == 0
            logits = eng.step([StepEntry(r, [t], [0], None if first else [i])
                               for i, (r, t) in enumerate(zip(rids, toks))])
            handle = sampler.sample_async(logits, params, counters, out=eng.feedback)
            if state["pending"] is not None:
                state["pending"].result()
            state["pending"], state["n"] = handle, state["n"] + 1
        for _ in range(warmup):
            one()
        state["pending"].result() if state["pending"] is not None else None
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(steps):
            one()
        state["pending"].result()                    # the last step's tokens have reached the host
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        ctx_tokens = batch * (start_ctx + warmup + steps / 2.0)
        for r in rids:
            eng.finish(r)
        return dt, ctx_tokens

    dt, ctx_tokens = decode_run(a.batch, a.steps, a.warmup)
    ms = dt / a.steps * 1e3
    value = a.batch * a.steps / dt
    nbytes = decode_bytes(cfg, a.layers, ctx_tokens, es)
    out = {
        "metric": f"decode tok/s (Qwen2-7B shape, batch {a.batch}, context {CONTEXT})", "value": round(value, 2),
        "unit": "tok/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": a.dtype,
        "data": "synthetic: seeded random token ids, random weights N(0, 0.02), random cache content",
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
                     "unit": "GB/s", "frac": round(nbytes / (ms * 1e-3) / HBM_PEAK, 4)},
    }
    if not a.no_prefill:
        prompt = rng.integers(0, cfg["vocab_size"], PREFILL_TOKENS).tolist()
        times = []
        for i in range(5):                           # one to warm up, the best of four
            torch.cuda.synchronize()
            t = time.perf_counter()
            logits = eng.step([StepEntry(f"p{i}", prompt, [PREFILL_TOKENS - 1])])
            sampler.sample(logits, [SamplingParams()], [0])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t)
            eng.finish(f"p{i}")
        pt = min(times[1:])
        out["prefill"] = {"value": round(PREFILL_TOKENS / pt, 1), "tokens": PREFILL_TOKENS,
                          "ms": round(pt * 1e3, 3),
                          "frac": round(prefill_flops(cfg, a.layers, PREFILL_TOKENS) / pt / FLOP_PEAK[a.dtype], 4)}
    if not a.no_points:
        pts = {}
        for b in (1, 64):
            d, _ = decode_run(b, max(8, a.steps // 2), 4)
            pts[f"decode_b{b}"] = round(b * max(8, a.steps // 2) / d, 2)
        out["points"] = pts
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
