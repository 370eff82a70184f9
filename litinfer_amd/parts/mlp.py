"""Dense SwiGLU feed-forward: y = (up * gate / (1 + exp(-gate))) Wd^T with
gate = xn Wg^T, up = xn Wu^T, no biases (src/llaisys/models/qwen2.cpp:744-759,
src/ops/swiglu/op.cpp:19-22).  Gate and up are one product with the packed
matrix [Wg; Wu]; the result is added to the residual stream."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import ParamSpec
from .base import BatchNeeds, FeedForward, register_part
from .linear import Linear


class SwiGLUMLP(FeedForward):
    graph_safe = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.hidden = int(spec.args["hidden_size"])
        self.inter = int(spec.args["intermediate_size"])
        self.gate_up = None
        self.down = None

    def expected_params(self):
        p = self.prefix
        return {p + "gate_proj.weight": ParamSpec((self.inter, self.hidden)),
                p + "up_proj.weight": ParamSpec((self.inter, self.hidden)),
                p + "down_proj.weight": ParamSpec((self.hidden, self.inter))}

    def batch_needs(self):
        return BatchNeeds(row_tile=self.down.row_tile() if self.down is not None else 1)

    def load_params(self, get):
        p = self.prefix
        g, u = get(p + "gate_proj.weight"), get(p + "up_proj.weight")
        dt = torch.float32 if torch.float32 in (g.dtype, u.dtype) else g.dtype
        self.gate_up = Linear(self.rt, torch.cat([g.to(dt), u.to(dt)], dim=0))
        self.down = Linear(self.rt, get(p + "down_proj.weight"))

    def forward_prenorm(self, norm, residual, xn, ctx):
        # few rows (decoding): the product before the norm may have left its rows scaled by the
        # norm's weights; the gate/up product then applies the rows' factors with its activation
        sc = residual.scaled_rows(norm)
        if sc is not None and self.gate_up.takes_swiglu(sc.rows):
            h = ctx.ws.buffer("mlp.h", (sc.rows.shape[0], self.inter), self.rt.dtype)
            self.gate_up(sc.rows, h, ws=ctx.ws, swiglu=True, row_scale=sc.scale)
            return residual.add_linear(self.down, h)
        self.forward(residual.normed(norm, xn), residual, ctx)

    def forward(self, xn, residual, ctx):
        t = xn.shape[0]
        h = ctx.ws.buffer("mlp.h", (t, self.inter), self.rt.dtype)
        if self.gate_up.takes_swiglu(xn):
            self.gate_up(xn, h, ws=ctx.ws, swiglu=True)        # few rows: the activation is the epilogue
        else:
            gu = ctx.ws.buffer("mlp.gate_up", (t, 2 * self.inter), self.rt.dtype)
            self.gate_up(xn, gu, ws=ctx.ws)
            ops.swiglu(gu, h)
        residual.add_linear(self.down, h)


register_part("feed_forward", "swiglu_mlp", SwiGLUMLP)
