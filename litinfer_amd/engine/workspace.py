"""Buffers that live across steps, so a step allocates nothing once the
largest batch has been seen."""
from __future__ import annotations

import math
from typing import Dict, Tuple

import torch


class Workspace:
    def __init__(self, device):
        self.device = torch.device(device)
        self._bufs: Dict[Tuple[str, torch.dtype], torch.Tensor] = {}
        self.generation = 0          # goes up whenever a buffer MOVES (is allocated anew, larger): recorded graphs are stale then
        self.allocations = 0         # goes up with every allocation, a name's first included
        self._views: Dict[Tuple[str, torch.dtype, Tuple[int, ...]], torch.Tensor] = {}

    def buffer(self, name: str, shape, dtype: torch.dtype, zero: bool = False) -> torch.Tensor:
        """A tensor of this shape; its contents are whatever the last user of
        the same name left.  `zero`: the buffer is zero when it is allocated (and
        again whenever it has to grow): for users that leave it as they found it."""
        shape = tuple(int(s) for s in shape)
        view = self._views.get((name, dtype, shape))
        if view is not None:                       # (asked for some hundred times a step, mostly with the same shapes)
            return view
        n = math.prod(shape)
        key = (name, dtype)
        buf = self._bufs.get(key)
        if buf is None or buf.numel() < max(1, n):
            cap = max(1, n) if buf is None else max(n, buf.numel() * 3 // 2)
            moved = buf is not None
            buf = (torch.zeros if zero else torch.empty)(cap, dtype=dtype, device=self.device)
            self._bufs[key] = buf
            self.allocations += 1
            if moved:                              # a name's first buffer moves nothing that a graph may have recorded
                self.generation += 1
            for k in [k for k in self._views if k[0] == name and k[1] is dtype]:
                del self._views[k]                 # views of the buffer that has just moved
        view = buf[:n].view(*shape)
        if len(self._views) < 4096:
            self._views[(name, dtype, shape)] = view
        return view
