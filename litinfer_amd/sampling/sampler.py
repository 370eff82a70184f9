"""Choosing next tokens: greedy, temperature, top-k, top-p.

The reference has three samplers that disagree (src/llaisys/models/qwen2.cpp:441-528
single path, :890-920 engine, python/llaisys/sampling.py); this one follows the
engine's filter order (temperature, then top-k, then top-p over the
survivors, then the softmax of what is left) and replaces its process-wide
generator (:1050) by a counter-based stream per request: the k-th sampled
token of a request uses uniform(seed, k), so a request's tokens do not depend
on what else is in the batch or on how the steps were cut.

Where the sampler is given the number of state slots, the options and the
stream of every live request lie in a table on the device, one row a slot
(the reference keeps them per sequence on the host,
src/llaisys/models/qwen2.hpp:100-110): `bind` writes a slot's row once, when a
request takes the slot, and `sample_bound_async` then needs one integer a row
from the host, the slot; the uniform numbers are drawn and counted on the
device.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np
import torch

from ..kernels import ops
from ..utils.pinned import BatchUploader

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


class PendingTokens:
    """Tokens that were chosen on the device and are on their way to the host."""

    def __init__(self, sampler, host: torch.Tensor, n: int, event):
        self._sampler, self._host, self._n, self._event = sampler, host, n, event
        self._tokens: Optional[List[int]] = None

    def result(self) -> List[int]:
        """The tokens; waits for the device if they are not there yet."""
        if self._tokens is None:
            if self._event is not None:
                self._event.synchronize()
            self._tokens = self._host[:self._n].tolist()
            self._sampler._give_back(self._host)
            self._host = None
        return self._tokens


class Sampler:
    def __init__(self, device, slots: int = 0):
        """slots: rows of the per-slot table on the device (the cache's state slots); 0: no table,
        every call brings its rows' options and counters from the host."""
        self.device = torch.device(device)
        self._free_host: List[torch.Tensor] = []
        self._params_up = None
        self.slots = int(slots)
        self.table = (torch.zeros((self.slots, ops.SAMPLE_SLOT_WORDS), dtype=torch.int32, device=self.device)
                      if self.slots > 0 else None)
        self._rows_up = None
        self._row_arrays = None

    # ---- the per-slot table -----------------------------------------------------
    def bind(self, slot: int, params: SamplingParams, draws: int = 0) -> None:
        """The request that holds state slot `slot` samples with `params`; `draws` numbers of its
        stream have been used already (a request that was preempted goes on where it was)."""
        if self.table is None or not 0 <= slot < self.slots:
            raise ValueError(f"sampler: no row for slot {slot} in a table of {self.slots}")
        seed = int(params.seed) & _MASK
        words = np.zeros(ops.SAMPLE_SLOT_WORDS, dtype=np.int32)
        words[0:2] = np.array([params.temperature if params.temperature > 0 else 0.0, params.top_p], dtype=np.float32).view(np.int32)
        words[2] = int(params.top_k)
        words[3:5] = np.array([seed & 0xffffffff, seed >> 32], dtype=np.uint32).view(np.int32)
        words[5] = int(draws)
        row = torch.from_numpy(words)
        if self.device.type == "cuda":
            row = row.pin_memory()
        self.table[slot].copy_(row, non_blocking=True)

    def sample_bound_async(self, logits: torch.Tensor, slots: Sequence[int], greedy: Sequence[bool],
                           out: Optional[torch.Tensor] = None) -> PendingTokens:
        """One token for each row of logits; row i belongs to the request in state slot slots[i], whose
        options and stream `bind` has written; greedy[i] makes the row greedy whatever the table says."""
        n = logits.shape[0]
        assert n == len(slots) == len(greedy) and self.table is not None
        if out is None:
            out = torch.empty(n, dtype=torch.int32, device=self.device)
        ids = out[:n]
        if all(greedy):
            ops.argmax_rows(logits, ids)
            return self._on_their_way(ids, n)
        rows = np.fromiter((s | (ops.SAMPLE_ROW_GREEDY if g else 0) for s, g in zip(slots, greedy)), dtype=np.int32, count=n)
        if self._rows_up is None:
            self._rows_up = BatchUploader(self.device)
        dev_rows = self._rows_up.upload([rows])[0]
        if self._row_arrays is None or self._row_arrays.shape[1] < n:
            self._row_arrays = torch.empty((4, max(n, 64)), dtype=torch.int32, device=self.device)
        a = self._row_arrays
        t, p, u, k = a[0, :n].view(torch.float32), a[1, :n].view(torch.float32), a[2, :n].view(torch.float32), a[3, :n]
        ops.sample_prepare(dev_rows, self.table, t, k, p, u)
        ops.sample_rows(logits, t, k, p, u, ids)
        return self._on_their_way(ids, n)

    def _on_their_way(self, ids: torch.Tensor, n: int) -> PendingTokens:
        hb = self._host_buffer(n)
        if self.device.type == "cuda":
            hb[:n].copy_(ids, non_blocking=True)
            ev = torch.cuda.Event()
            ev.record()
        else:
            hb[:n].copy_(ids)
            ev = None
        return PendingTokens(self, hb, n, ev)

    def _host_buffer(self, n: int) -> torch.Tensor:
        for i, b in enumerate(self._free_host):
            if b.numel() >= n:
                return self._free_host.pop(i)
        return torch.empty(max(n, 256), dtype=torch.int32, pin_memory=self.device.type == "cuda")

    def _give_back(self, buf: torch.Tensor) -> None:
        if len(self._free_host) < 8:
            self._free_host.append(buf)

    def sample_async(self, logits: torch.Tensor, params: Sequence[SamplingParams], counters: Sequence[int],
                     out: Optional[torch.Tensor] = None) -> PendingTokens:
        """One token for each row of logits [n, vocab] (float32, on the device),
        written to out[:n] (int32, on the device; e.g. the engine's feedback
        buffer, from which the next step can take them) and copied to the host
        without waiting: `result()` of what is returned waits and gives the list."""
        n = logits.shape[0]
        assert n == len(params) == len(counters)
        if out is None:
            out = torch.empty(n, dtype=torch.int32, device=self.device)
        assert out.dtype is torch.int32 and out.numel() >= n and out.device == logits.device
        ids = out[:n]
        if all(p.greedy for p in params):
            ops.argmax_rows(logits, ids)
        else:
            host = np.empty((4, n), dtype=np.float32)
            host[0] = [p.temperature if p.temperature > 0 else 0.0 for p in params]
            host[1] = [p.top_p for p in params]
            host[2] = [uniform(p.seed, c) for p, c in zip(params, counters)]
            host[3] = np.array([p.top_k for p in params], dtype=np.int32).view(np.float32)
            if self._params_up is None:
                self._params_up = BatchUploader(self.device)       # pinned, so the copy does not wait for the stream
            dev = self._params_up.upload([host.view(np.int32)])[0]
            f = dev.view(torch.float32)
            ops.sample_rows(logits, f[0], dev[3], f[1], f[2], ids)
        return self._on_their_way(ids, n)

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams],
               counters: Sequence[int]) -> List[int]:
        """One token for each row of logits [n, vocab] (float32, on the device)."""
        return self.sample_async(logits, params, counters).result()
