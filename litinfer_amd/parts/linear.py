"""A weight matrix [out, in] with an optional bias: y = x W^T + b
(src/ops/linear/cpu/linear_cpu.cpp:32-37).  Not a part of its own in a layer;
mixers, feed-forwards and the head hold these."""
from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops


class Linear:
    def __init__(self, rt, weight: torch.Tensor, bias: Optional[torch.Tensor] = None):
        self.rt = rt
        self.weight = rt.matrix(weight)      # the same buffer when it already is as needed
        self.bias = None if bias is None else rt.vector(bias)
        self.out_features, self.in_features = self.weight.shape

    def row_tile(self) -> int:
        """Rows that the kernels of this product take at a time (for `BatchNeeds.row_tile`)."""
        return ops.linear_row_tile(self.rt.dtype) if self.rt.device.type == "cuda" else 1

    def takes_swiglu(self, x: torch.Tensor) -> bool:
        """Whether the product of these rows can have the SwiGLU activation as its
        epilogue (no bias, x and the matrix of one dtype, a size the kernels take)."""
        return (x.dtype is self.weight.dtype and self.bias is None and x.data_ptr() % 16 == 0
                and ops.swiglu_takes(x.shape[0], self.in_features, self.weight.dtype))

    def takes_scaling(self, x: torch.Tensor, out: torch.Tensor) -> bool:
        """Whether out += x W^T + b can also leave out times a norm's weights and the
        shares of the rows' sums of squares (few rows, bfloat16 operands)."""
        return (x.dtype is torch.bfloat16 and out.dtype is torch.float32
                and ops.few_rows_preferred(x.shape[0], self.out_features, self.in_features)
                and ops.residual_norm_takes(x.shape[0], self.out_features, self.in_features, self.weight.dtype))

    def add_with_scaling(self, x: torch.Tensor, out: torch.Tensor, scaling, rows: torch.Tensor, ws):
        """out += x W^T + b; rows = scaling.weight * out.  Returns what the product
        behind the norm needs for the rows' factors."""
        parts = ws.buffer("linear.sq_parts", (ops.RESIDUAL_NORM_MAX_PARTS * ops.RESIDUAL_NORM_MAX_ROWS,), torch.float32)
        n = ops.linear_residual_norm(x, self.weight, self.bias, out, scaling.weight, rows, parts)
        return ops.RowScale(parts, n, scaling.eps)

    def add_then_norm(self, x: torch.Tensor, out: torch.Tensor, scaling, xn: torch.Tensor, ws) -> bool:
        """out += x W^T + b and xn = the RMS norm of the new out, in one go where the
        kernels have that (a product cut along K); False, with nothing done, where not."""
        if self.weight.dtype is not torch.bfloat16 or x.dtype is not torch.bfloat16 or out.dtype is not torch.float32:
            return False
        return ops.linear_then_norm(x, self.weight, self.bias, out, scaling.weight, scaling.eps, xn, ws)

    def __call__(self, x: torch.Tensor, out: torch.Tensor, accumulate: bool = False, ws=None,
                 swiglu: bool = False, row_scale=None):
        """out = x W^T + b, or out += ... when `accumulate` (out is float32 then).
        With `swiglu` (only where `takes_swiglu`) W is [gate; up] and out gets
        up * silu(gate); `row_scale` then says that x came out of `add_with_scaling`.  A matrix that is stored in 32-bit is multiplied in
        32-bit also when the activations are bfloat16: they are widened for it,
        exactly."""
        if swiglu:
            ops.linear_swiglu(x, self.weight, out, row_scale=row_scale)
        elif self.weight.dtype is torch.float32 and x.dtype is not torch.float32:
            x32 = ws.buffer("linear.x32", x.shape, torch.float32)
            ops.cast(x, x32)
            if out.dtype is torch.float32:
                ops.linear(x32, self.weight, self.bias, out, accumulate, ws=ws)
            else:
                y32 = ws.buffer("linear.y32", out.shape, torch.float32)
                ops.linear(x32, self.weight, self.bias, y32, False)
                ops.cast(y32, out)
        else:
            ops.linear(x, self.weight, self.bias, out, accumulate, ws=ws)      # few rows go to their own kernels inside
        return out
