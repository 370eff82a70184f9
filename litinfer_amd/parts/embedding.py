"""Token embedding and the output head.

Embedding: x[t, :] = E[ids[t], :], a row copy without scaling
(src/ops/embedding/op.cpp:32-40), written into the float32 residual stream.
Head: logits = xf Wout^T without bias (src/llaisys/models/qwen2.cpp:337), as
float32; when tied, Wout is the embedding table itself (one buffer), and so it
is when the configuration says untied but the checkpoint holds no head matrix
(python/llaisys/models/qwen2.py:196-199)."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import ParamSpec
from .base import Part, register_part
from .linear import Linear


class TokenEmbedding(Part):
    graph_safe = True

    category = "embedding"

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.vocab = int(spec.args["vocab_size"])
        self.hidden = int(spec.args["hidden_size"])
        self.table = None

    def expected_params(self):
        return {self.prefix + "weight": ParamSpec((self.vocab, self.hidden))}

    def load_params(self, get):
        self.table = self.rt.matrix(get(self.prefix + "weight"))

    def forward(self, ids, out, id_src=None, feedback=None):
        ops.embedding(ids, self.table, out, id_src, feedback)
        return out


class LinearHead(Part):
    graph_safe = True

    category = "head"

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.vocab = int(spec.args["vocab_size"])
        self.hidden = int(spec.args["hidden_size"])
        self.tied_to = spec.args.get("tied_to")
        # untied by the configuration, but no matrix stored: use the table, as the reference does
        self.tie_if_absent = bool(spec.args.get("tie_if_absent", False))
        self.proj = None

    def expected_params(self):
        if self.tied_to:
            return {}
        return {self.prefix + "weight": ParamSpec((self.vocab, self.hidden), required=not self.tie_if_absent)}

    def load_params(self, get, tied_table=None):
        """`tied_table` is the embedding's table as the model holds it."""
        w = None if self.tied_to else get(self.prefix + "weight")
        if w is None:
            if tied_table is None:
                raise ValueError("head: tied to the embedding, but no table was given")
            if not self.tied_to and hasattr(get, "note"):
                get.note(f"{self.prefix}weight is not stored: the head uses the embedding table")
            self.proj = Linear(self.rt, tied_table)
        else:
            self.proj = Linear(self.rt, w)

    def forward(self, xn, out, ws):
        return self.proj(xn, out, ws=ws)


register_part("embedding", "token_embedding", TokenEmbedding)
register_part("head", "linear_head", LinearHead)
