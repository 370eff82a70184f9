"""The residual stream of a step: a float32 tensor [T, H] that the parts of a
layer add into, in 32-bit.

Parts do not add by themselves; they ask the stream: `add_linear(linear, h)`
adds `h W^T + b`, `normed(norm, out)` gives the norm of the current sum, and
`tensor()` gives the sum itself (for a part that wants to add something of its
own).  That lets the stream choose how a sum is carried out.  When decoding, a
product with few output columns is cut along K over many blocks so that every
compute unit streams an equal share of the matrix; its partial sums are then
added up, added to the stream and normed for the next part in ONE kernel
instead of three (src/llaisys/models/qwen2.cpp:287-297 does linear, add and
rms_norm as three passes).
"""
from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops


class ResidualStream:
    def __init__(self, x: torch.Tensor, ws):
        self.x = x
        self.ws = ws
        self._pending = None            # (partial sums [parts, T, H], bias) not yet added to x

    @property
    def shape(self):
        return self.x.shape

    def tensor(self) -> torch.Tensor:
        """The sum so far, with everything added."""
        self._flush()
        return self.x

    def add_linear(self, linear, h: torch.Tensor) -> None:
        """x += h W^T + b."""
        self._flush()
        parts = linear.split_parts(h)
        if parts > 1:
            partial = self.ws.buffer("stream.partial", (parts, h.shape[0], linear.out_features), torch.float32)
            ops.linear_skinny(h, linear.weight, None, partial, parts=parts)
            self._pending = (partial, linear.bias)
        else:
            linear(h, self.x, accumulate=True, ws=self.ws)

    def normed(self, norm, out: torch.Tensor) -> torch.Tensor:
        """out = norm(x)."""
        if self._pending is not None and getattr(norm, "fusable_rmsnorm", False):
            partial, bias = self._pending
            self._pending = None
            ops.skinny_finish(partial, bias, self.x, norm.weight, norm.eps, out)
        else:
            self._flush()
            norm.forward(self.x, out)
        return out

    def _flush(self) -> None:
        if self._pending is not None:
            partial, bias = self._pending
            self._pending = None
            ops.skinny_finish(partial, bias, self.x)
