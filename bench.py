#!/usr/bin/env python3
"""Decode and prefill throughput of the engine at the Qwen2-7B layer sizes (and, with
--mode serving | long, the other two measured workloads).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L] [--dtype bf16|fp32]

The measurements themselves are `litinfer_amd/benchmark.py` (also reachable as
`python -m litinfer_amd bench`); one JSON line is printed.
"""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

from litinfer_amd.benchmark import main  # noqa: E402

if __name__ == "__main__":
    sys.exit(main())
