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
        self.generation = 0          # goes up whenever a buffer moves: recorded graphs are stale then

    def buffer(self, name: str, shape, dtype: torch.dtype) -> torch.Tensor:
        """A tensor of this shape; its contents are whatever the last user of
        the same name left."""
        n = max(1, math.prod(int(s) for s in shape))
        key = (name, dtype)
        buf = self._bufs.get(key)
        if buf is None or buf.numel() < n:
            cap = n if buf is None else max(n, buf.numel() * 3 // 2)
            buf = torch.empty(cap, dtype=dtype, device=self.device)
            self._bufs[key] = buf
            self.generation += 1
        return buf[:math.prod(int(s) for s in shape)].view(*shape)
