"""Grouped-query attention over the paged cache.

q = xn Wq^T + bq, k, v likewise (src/llaisys/models/qwen2.cpp:613-615); the
position encoding acts on q and k only (:628-629); keys and values are written
to their pages before the attention, so a portion attends to itself through
the cache (:659-690); query head h reads kv head h // (heads/kv_heads), the
query at position p sees keys t <= p, and with a window only p - t < window
(src/ops/paged_attention/op.cpp:20-64); scale 1/sqrt(head_dim) unless given
(:690 of qwen2.cpp); output projection (:699), added to the residual stream.
The three projections are one product with a packed matrix [Wq; Wk; Wv].
"""
from __future__ import annotations

import math

import torch

from ..kernels import ops
from ..weights.loader import ParamSpec
from .base import BatchNeeds, Mixer, PagedKVNeed, build_part, register_part
from .linear import Linear


class GQAttention(Mixer):

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        a = spec.args
        self.hidden = int(a["hidden_size"])
        self.nh = int(a["num_heads"])
        self.nkv = int(a["num_kv_heads"])
        self.dh = int(a["head_dim"])
        self.window = int(a.get("window") or 0)
        self.qkv_bias = bool(a.get("qkv_bias", False))
        self.out_bias = bool(a.get("out_bias", False))
        self.scale = float(a["scale"]) if a.get("scale") is not None else 1.0 / math.sqrt(self.dh)
        if self.nh % self.nkv:
            raise ValueError(f"attention: {self.nh} heads are not a multiple of {self.nkv} kv heads")
        ops.check_attention_sizes(self.nh, self.nkv, self.dh)
        self.position = build_part("position", a["position"], rt) if a.get("position") else None
        self.n_q = self.nh * self.dh
        self.n_kv = self.nkv * self.dh
        self.qkv = None
        self.out = None

    @property
    def graph_safe(self):
        return self.position is None or self.position.graph_safe

    def cache_need(self):
        return PagedKVNeed(self.nkv, self.dh, self.window)

    def batch_needs(self):
        # the kernels take single-token segments (split keys) and the others (tiles of queries) apart
        return BatchNeeds(tile_rows=ops.PREFILL_TILE_ROWS, token_kinds=True,
                          row_tile=self.qkv.row_tile() if self.qkv is not None else 1)

    def expected_params(self):
        p = self.prefix
        e = {p + "q_proj.weight": ParamSpec((self.n_q, self.hidden)),
             p + "k_proj.weight": ParamSpec((self.n_kv, self.hidden)),
             p + "v_proj.weight": ParamSpec((self.n_kv, self.hidden)),
             p + "o_proj.weight": ParamSpec((self.hidden, self.n_q))}
        if self.qkv_bias:   # used when present, skipped when absent (src/ops/linear/op.cpp:55)
            e[p + "q_proj.bias"] = ParamSpec((self.n_q,), required=False)
            e[p + "k_proj.bias"] = ParamSpec((self.n_kv,), required=False)
            e[p + "v_proj.bias"] = ParamSpec((self.n_kv,), required=False)
        if self.out_bias:
            e[p + "o_proj.bias"] = ParamSpec((self.hidden,), required=False)
        return e

    def load_params(self, get):
        p = self.prefix
        ws = [get(p + f"{n}_proj.weight") for n in "qkv"]
        dt = torch.float32 if any(w.dtype is torch.float32 for w in ws) else ws[0].dtype
        w = torch.cat([x.to(dt) for x in ws], dim=0)
        b = None
        if self.qkv_bias:
            bs = [get(p + f"{n}_proj.bias") for n in "qkv"]
            if any(x is not None for x in bs):
                sizes = (self.n_q, self.n_kv, self.n_kv)
                b = torch.cat([torch.zeros(s) if x is None else x.to(torch.float32)
                               for x, s in zip(bs, sizes)])
        self.qkv = Linear(self.rt, w, b)
        self.out = Linear(self.rt, get(p + "o_proj.weight"),
                          get(p + "o_proj.bias") if self.out_bias else None)

    def forward_prenorm(self, norm, residual, xn, ctx, cache):
        # few rows (decoding): the product before the norm may have left its rows scaled by the
        # norm's weights; then projection, rows' factors, encoding and page write are one kernel
        sc = residual.scaled_rows(norm)
        if sc is not None and self.position is not None:
            qkv = ctx.ws.buffer("attn.qkv", (sc.rows.shape[0], self.n_q + 2 * self.n_kv), self.rt.dtype)
            if self.position.project_encode_store(self.qkv, sc.rows, qkv, self.nh, self.nkv, self.dh, ctx, cache,
                                                  row_scale=sc.scale):
                return self._attend(qkv, residual, ctx, cache)
        self.forward(residual.normed(norm, xn), residual, ctx, cache)

    def forward(self, xn, residual, ctx, cache):
        t = xn.shape[0]
        qkv = ctx.ws.buffer("attn.qkv", (t, self.n_q + 2 * self.n_kv), self.rt.dtype)
        fused = self.position is not None and self.position.project_encode_store(
            self.qkv, xn, qkv, self.nh, self.nkv, self.dh, ctx, cache)
        if not fused:                                # else projection, encoding and page write were one kernel
            self.qkv(xn, qkv, ws=ctx.ws)
            if self.position is not None:
                self.position.encode_and_store(qkv, self.nh, self.nkv, self.dh, ctx, cache)
            elif cache.owned:
                ops.kv_store(qkv, self.nh, self.nkv, self.dh, ctx.slot_map(cache.group),
                             cache.k, cache.v, cache.page_size)
        self._attend(qkv, residual, ctx, cache)

    def _attend(self, qkv, residual, ctx, cache):
        attn = ctx.ws.buffer("attn.out", (qkv.shape[0], self.n_q), self.rt.dtype)
        ops.paged_attention(qkv, attn, cache.k, cache.v, ctx.attention_meta(cache.group),
                            self.nh, self.nkv, self.dh, cache.page_size, self.window, self.scale, ws=ctx.ws)
        residual.add_linear(self.out, attn)


register_part("mixer", "gqa_attention", GQAttention)
