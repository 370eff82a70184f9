"""The residual stream of a step: a float32 tensor [T, H] that the parts of a
layer add into, in 32-bit.

Parts do not add by themselves; they ask the stream: `add_linear(linear, h)`
adds `h W^T + b` (the product kernel's epilogue does the add in 32-bit, so no
separate pass reads and writes the stream: src/llaisys/models/qwen2.cpp:287-290
does linear and add as two), `normed(norm, out)` gives the norm of the current
sum, and `tensor()` gives the sum itself for a part that adds in its own way.
"""
from __future__ import annotations

import torch


class ResidualStream:
    def __init__(self, x: torch.Tensor, ws):
        self.x = x
        self.ws = ws

    @property
    def shape(self):
        return self.x.shape

    def tensor(self) -> torch.Tensor:
        """The sum so far."""
        return self.x

    def add_linear(self, linear, h: torch.Tensor) -> None:
        """x += h W^T + b."""
        linear(h, self.x, accumulate=True, ws=self.ws)

    def normed(self, norm, out: torch.Tensor) -> torch.Tensor:
        """out = norm(x)."""
        norm.forward(self.x, out)
        return out
