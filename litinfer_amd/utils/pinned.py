"""Small integer arrays from the host to the device in one copy that does not wait."""
from __future__ import annotations

from typing import List

import numpy as np
import torch


class BatchUploader:
    """Packs the step's integers into pinned host memory and copies them to
    the device once.  Two host buffers alternate, each guarded by an event, so
    a buffer is not rewritten while its copy may still be in flight."""

    def __init__(self, device):
        self.device = torch.device(device)
        self._host = [None, None]
        self._events = [None, None]
        self._dev = None
        self._turn = 0
        self.generation = 0          # goes up when the device buffer moves

    def stage(self, total: int) -> torch.Tensor:
        """A pinned host buffer of at least `total` int32 words to be filled and then sent with
        `push`; waits until that buffer's last copy has left it."""
        total = max(int(total), 4)
        i = self._turn
        if self._host[i] is None or self._host[i].numel() < total:
            self._host[i] = torch.empty(total * 2, dtype=torch.int32, pin_memory=self.device.type == "cuda")
        elif self._events[i] is not None:
            self._events[i].synchronize()
        return self._host[i]

    def push(self, total: int) -> torch.Tensor:
        """Copy the first `total` words of the staged buffer to the device (without waiting)
        and return the device buffer."""
        total = max(int(total), 4)
        i = self._turn
        self._turn ^= 1
        if self._dev is None or self._dev.numel() < total:
            self._dev = torch.empty(max(total * 2, 1 << 16), dtype=torch.int32, device=self.device)
            self.generation += 1
        if self.device.type == "cuda":
            # a fresh device buffer per step would be simpler; one buffer is enough because the
            # copy is ordered on the stream after the kernels of the step before
            self._dev[:total].copy_(self._host[i][:total], non_blocking=True)
            ev = torch.cuda.Event()
            ev.record()
            self._events[i] = ev
        else:
            self._dev[:total].copy_(self._host[i][:total])
        return self._dev

    def upload(self, parts: List[np.ndarray]) -> List[torch.Tensor]:
        offs, total = [], 0
        for p in parts:
            offs.append(total)
            total += (p.size + 3) // 4 * 4            # 16-byte alignment of every array
        h = self.stage(total).numpy()
        for p, o in zip(parts, offs):
            h[o:o + p.size] = p.reshape(-1)
        dev = self.push(total)
        return [dev[o:o + p.size].view(p.shape) for p, o in zip(parts, offs)]
