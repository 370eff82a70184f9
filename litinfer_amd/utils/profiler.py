"""Timing by operator and a per-step trace, switched on from the environment as
in the reference: LLAISYS_PROFILE=1 (src/utils/profiler.cpp:48-55: "1", "true",
"on") records the time of every kernel call under the current phase (prefill /
decode) and prints a table when the process ends (:70-110); LLAISYS_TRACE=1
(src/llaisys/models/qwen2.cpp:17-24) prints one line per step.

The reference times its CPU operators as they run; on the GPU a call only
enqueues work, so with the profiler on every call is followed by a wait for the
device and recorded steps are not used: the times are those of the kernels one
by one, not of a step at full speed."""
from __future__ import annotations

import atexit
import os
import sys
import time
from collections import defaultdict
from typing import Dict, Tuple

_ON = ("1", "true", "on")


def _flag(name: str) -> bool:
    return os.environ.get(name, "").strip().lower() in _ON


def trace_enabled() -> bool:
    return _flag("LLAISYS_TRACE")


class OpProfiler:
    def __init__(self, enabled: bool):
        self.enabled = enabled
        self.phase = ""
        self.total: Dict[Tuple[str, str], float] = defaultdict(float)
        self.calls: Dict[Tuple[str, str], int] = defaultdict(int)
        if enabled:
            atexit.register(self.report)

    def record(self, name: str, seconds: float) -> None:
        key = (self.phase, name)
        self.total[key] += seconds
        self.calls[key] += 1

    def timed(self, name: str, launch, sync) -> None:
        """Run `launch()` between two waits for the device and record it."""
        sync()
        t = time.perf_counter()
        launch()
        sync()
        self.record(name, time.perf_counter() - t)

    def report(self, out=None) -> None:
        if not self.total:
            return
        out = out or sys.stderr
        whole = sum(self.total.values())
        print("[litinfer_amd profile] operator times (each call waited for)", file=out)
        print(f"{'phase':8s} {'operator':32s} {'calls':>8s} {'total ms':>11s} {'avg us':>10s} {'share':>7s}", file=out)
        for (phase, name), sec in sorted(self.total.items(), key=lambda kv: -kv[1]):
            n = self.calls[(phase, name)]
            print(f"{phase or '-':8s} {name:32s} {n:8d} {sec * 1e3:11.3f} {sec / n * 1e6:10.1f} "
                  f"{sec / whole * 100:6.2f}%", file=out)
        out.flush()


profiler = OpProfiler(_flag("LLAISYS_PROFILE"))
