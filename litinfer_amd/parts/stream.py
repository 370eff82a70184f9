"""The residual stream of a step: a float32 tensor [T, H] that the parts of a
layer add into, in 32-bit.

Parts do not add by themselves; they ask the stream: `add_linear(linear, h)`
adds `h W^T + b` (the product kernel's epilogue does the add in 32-bit, so no
separate pass reads and writes the stream: src/llaisys/models/qwen2.cpp:287-290
does linear and add as two), `normed(norm, out)` gives the norm of the current
sum, and `tensor()` gives the sum itself for a part that adds in its own way.

Whoever knows which norm reads the stream next says so in `next_norm`.  Then
`add_linear` may, for the few rows of a decoding step, have its kernel leave the
sum times that norm's weights and the rows' sums of squares beside the sum
itself, and the part behind the norm finds them under `scaled_rows(norm)`: the
norm costs no pass of its own.  Any other write to the stream forgets them.
"""
from __future__ import annotations

from typing import Optional

import torch

from .base import ScaledRows


class ResidualStream:
    def __init__(self, x: torch.Tensor, ws):
        self.x = x
        self.ws = ws
        self.next_norm = None                 # the norm through which the stream is read next, if known
        self._scaled = None                   # (norm, ScaledRows) left by the last add_linear
        self._normed = None                   # (norm, its result) left by the last add_linear

    @property
    def shape(self):
        return self.x.shape

    def tensor(self) -> torch.Tensor:
        """The sum so far (whoever takes it may write to it)."""
        self._scaled = self._normed = None
        return self.x

    def add_linear(self, linear, h: torch.Tensor) -> None:
        """x += h W^T + b."""
        norm, self._scaled, self._normed = self.next_norm, None, None
        scaling = norm.as_scaling() if norm is not None else None
        if scaling is not None and linear.takes_scaling(h, self.x):
            rows = self.ws.buffer("stream.scaled_rows", self.x.shape, h.dtype)
            self._scaled = (norm, ScaledRows(rows, linear.add_with_scaling(h, self.x, scaling, rows, self.ws)))
            return
        if scaling is not None:
            # some more rows: where the product is cut along K, the kernel that adds the parts up norms as well
            rows = self.ws.buffer("stream.normed_rows", self.x.shape, h.dtype)
            if linear.add_then_norm(h, self.x, scaling, rows, self.ws):
                self._normed = (norm, rows)
                return
        linear(h, self.x, accumulate=True, ws=self.ws)

    def scaled_rows(self, norm) -> Optional[ScaledRows]:
        """What the last addition left for this norm's reader, if it did."""
        if self._scaled is not None and self._scaled[0] is norm:
            return self._scaled[1]
        return None

    def normed(self, norm, out: torch.Tensor) -> torch.Tensor:
        """norm(x): in `out`, or in the tensor that the last addition already left."""
        if self._normed is not None and self._normed[0] is norm:
            return self._normed[1]
        norm.forward(self.x, out)
        return out
