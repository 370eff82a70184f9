"""Schedules: ways of cutting the same requests into steps.

A schedule is a list of steps; a step is (entries, end) with entries a list of
(request id, first token index, number of tokens) and end a list of request
ids that are finished after the step.  Every token's logits are asked for, so
all schedules of the same requests give comparable [len, vocab] arrays.
"""
from __future__ import annotations

from typing import Dict, List, Sequence, Tuple

import numpy as np

Step = Tuple[List[Tuple[str, int, int]], List[str]]


def whole(requests: Dict[str, Sequence[int]]) -> List[Step]:
    """Each request alone, all its tokens in one step."""
    return [([(rid, 0, len(t))], [rid]) for rid, t in requests.items()]


def tail(requests, n_tail=32) -> List[Step]:
    """Each request alone: most of it in one step, the last n_tail tokens one by one."""
    steps = []
    for rid, t in requests.items():
        n = len(t)
        head = max(1, n - n_tail) if n > 1 else 1
        steps.append(([(rid, 0, head)], [rid] if head == n else []))
        for i in range(head, n):
            steps.append(([(rid, i, 1)], [rid] if i == n - 1 else []))
    return steps


CHUNK_CYCLE = (7, 2, 13, 3, 2, 24, 5, 1, 16, 2, 9)


def chunks(requests, cycle=CHUNK_CYCLE) -> List[Step]:
    """Each request alone in portions of changing size, down to two tokens and one."""
    steps = []
    for k, (rid, t) in enumerate(requests.items()):
        i, c = 0, k
        while i < len(t):
            n = min(cycle[c % len(cycle)], len(t) - i)
            steps.append(([(rid, i, n)], [rid] if i + n == len(t) else []))
            i += n
            c += 1
    return steps


def mixed(requests, max_live=4, seed=0, prefill_chunks=(24, 7, 2, 13, 5), decode_after=0.6) -> List[Step]:
    """Up to max_live requests at a time: each first goes through part of its
    tokens in portions (as a prompt would), then one token per step (as decoding
    would); portions of some stand beside single tokens of others; now and then a
    request sits a step out.  A finished request is ended at once and the next
    one starts, so its pages are taken again."""
    rng = np.random.default_rng(seed)
    waiting = list(requests.items())
    live: List[dict] = []
    steps: List[Step] = []
    c = 0
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, t = waiting.pop(0)
            live.append({"rid": rid, "n": len(t), "i": 0, "prompt": max(1, int(len(t) * decode_after))})
            if rng.random() < 0.5:
                break                              # staggered starts
        entries, end = [], []
        for r in live:
            if len(live) > 1 and rng.random() < 0.15:
                continue                           # sits this step out
            if r["i"] < r["prompt"]:
                n = min(prefill_chunks[c % len(prefill_chunks)], r["prompt"] - r["i"])
                c += 1
            else:
                n = 1
            entries.append((r["rid"], r["i"], n))
            r["i"] += n
            if r["i"] == r["n"]:
                end.append(r["rid"])
        if not entries:
            continue
        live = [r for r in live if r["rid"] not in end]
        steps.append((entries, end))
    return steps


def max_live_tokens(requests, steps: List[Step], round_to=64) -> int:
    """The most tokens live requests hold at any time, each rounded up to a
    multiple of round_to."""
    have: Dict[str, int] = {}
    worst = 0
    for entries, end in steps:
        for rid, i, n in entries:
            have[rid] = i + n
        worst = max(worst, sum(-(-v // round_to) * round_to for v in have.values()))
        for rid in end:
            have.pop(rid, None)
    return worst


def run(engine, requests, steps: List[Step]) -> Dict[str, np.ndarray]:
    """Drive the engine's step function through a schedule; returns the logits
    of every token of every request."""
    from litinfer_amd.engine import StepEntry
    rows: Dict[str, List[np.ndarray]] = {rid: [] for rid in requests}
    for entries, end in steps:
        batch = [StepEntry(rid, list(requests[rid][i:i + n]), list(range(n))) for rid, i, n in entries]
        logits = engine.step(batch).float().cpu().numpy()
        o = 0
        for rid, i, n in entries:
            rows[rid].append(logits[o:o + n])
            o += n
        for rid in end:
            engine.finish(rid)
    return {rid: np.concatenate(v) for rid, v in rows.items() if v}


def rel_err(got: np.ndarray, ref: np.ndarray) -> float:
    return float(np.abs(got.astype(np.float64) - ref).max() / np.abs(ref).max())


def mean_err(got: np.ndarray, ref: np.ndarray) -> float:
    """The mean deviation over all logits, in units of the largest logit: rounding scatters around zero and
    leaves this far below the largest deviation, a defect that moves every logit a little does not."""
    return float(np.abs(got.astype(np.float64) - ref).mean() / np.abs(ref).max())
