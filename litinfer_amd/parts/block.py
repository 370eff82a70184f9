"""The pre-norm arrangement of a layer's parts
(src/llaisys/models/qwen2.cpp:272-317): x += mixer(norm1(x)); x += ffn(norm2(x)).
The residual stream x is float32; mixer and feed-forward add into it through
the `ResidualStream` they are given."""
from __future__ import annotations

from .base import Block, build_part, register_part


class PreNormBlock(Block):
    def __init__(self, spec, rt, parts):
        super().__init__(spec, rt)
        self.norm1 = build_part("norm", parts["norm1"], rt)
        self.mixer = build_part("mixer", parts["mixer"], rt)
        self.norm2 = build_part("norm", parts["norm2"], rt)
        self.ffn = build_part("feed_forward", parts["feed_forward"], rt)
        self._all = (self.norm1, self.mixer, self.norm2, self.ffn)

    @property
    def graph_safe(self):
        return all(p.graph_safe for p in self._all)

    def cache_need(self):
        return self.mixer.cache_need()

    def batch_needs(self):
        needs = super().batch_needs()
        for p in self._all:
            needs = needs.merged(p.batch_needs())
        return needs

    def expected_params(self):
        e = {}
        for p in self._all:
            e.update(p.expected_params())
        return e

    def load_params(self, get):
        for p in self._all:
            p.load_params(get)

    def first_norm(self):
        return self.norm1

    def forward(self, stream, ctx, cache):
        xn = ctx.ws.buffer("block.xn", stream.shape, self.rt.dtype)
        after = stream.next_norm                   # the norm that reads the stream after this block
        stream.next_norm = self.norm2
        self.mixer.forward_prenorm(self.norm1, stream, xn, ctx, cache)
        stream.next_norm = after
        self.ffn.forward_prenorm(self.norm2, stream, xn, ctx)
        stream.next_norm = None


register_part("block", "prenorm", PreNormBlock)
