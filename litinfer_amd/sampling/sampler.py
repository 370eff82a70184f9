"""Choosing next tokens: greedy, temperature, top-k, top-p.

The reference has three samplers that disagree (src/llaisys/models/qwen2.cpp:441-528
single path, :890-920 engine, python/llaisys/sampling.py); this one follows the
engine's filter order (temperature, then top-k, then top-p over the
survivors, then the softmax of what is left) and replaces its process-wide
generator (:1050) by a counter-based stream per request: the k-th sampled
token of a request uses uniform(seed, k), so a request's tokens do not depend
on what else is in the batch or on how the steps were cut.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Sequence

import numpy as np
import torch

from ..kernels import ops

_MASK = (1 << 64) - 1


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0        # <= 0: greedy (src/llaisys/models/qwen2.cpp:893-895)
    top_k: int = 0                  # active when 0 < top_k < vocabulary (:903)
    top_p: float = 1.0              # active when 0 < top_p < 1 (:904)
    seed: int = 0

    @property
    def greedy(self) -> bool:
        return not self.temperature > 0.0


def uniform(seed: int, counter: int) -> float:
    """The counter-th number of the stream `seed`: a splitmix64 hash of both,
    its upper 24 bits as a float32-exact value in [0, 1)."""
    z = (seed * 0x9E3779B97F4A7C15 + (counter + 1) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    z ^= z >> 31
    return (z >> 40) / float(1 << 24)


class Sampler:
    def __init__(self, device):
        self.device = torch.device(device)

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams],
               counters: Sequence[int]) -> List[int]:
        """One token for each row of logits [n, vocab] (float32, on the device)."""
        n = logits.shape[0]
        assert n == len(params) == len(counters)
        out = torch.empty(n, dtype=torch.int32, device=self.device)
        if all(p.greedy for p in params):
            ops.argmax_rows(logits, out)
            return out.tolist()
        host = np.empty((4, n), dtype=np.float32)
        host[0] = [p.temperature if p.temperature > 0 else 0.0 for p in params]
        host[1] = [p.top_p for p in params]
        host[2] = [uniform(p.seed, c) for p, c in zip(params, counters)]
        topk = np.array([p.top_k for p in params], dtype=np.int32)
        host[3] = topk.view(np.float32)
        dev = torch.from_numpy(host).to(self.device)
        ops.sample_rows(logits, dev[0], dev[3].view(torch.int32), dev[1], dev[2], out)
        return out.tolist()
