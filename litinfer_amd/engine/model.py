"""A model built from a ModelSpec: embedding, layers in an execution order,
final norm, head.  It knows parts only through their interfaces."""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from ..config.spec import ModelSpec, PartSpec
from ..kernels import ops
from ..parts.base import Runtime, build_part
from ..parts.stream import ResidualStream
from ..weights.loader import ParamSpec


class Model:
    def __init__(self, spec: ModelSpec, rt: Runtime):
        spec.validate()
        self.spec = spec
        self.rt = rt
        self.embedding = build_part("embedding", spec.embedding, rt)
        self.layers = [build_part("block", PartSpec(l.block), rt, parts=l.parts) for l in spec.layers]
        self.final_norm = build_part("norm", spec.final_norm, rt)
        self.head = build_part("head", spec.head, rt)
        self.order = list(spec.order)
        self._batch_needs = None

    # ---- weights ----------------------------------------------------------
    def expected_params(self) -> Dict[str, ParamSpec]:
        e: Dict[str, ParamSpec] = {}
        for p in (self.embedding, *self.layers, self.final_norm, self.head):
            e.update(p.expected_params())
        return e

    def load_params(self, get) -> None:
        self._batch_needs = None                     # parts may answer differently once they hold their tensors
        self.embedding.load_params(get)
        for layer in self.layers:
            layer.load_params(get)
        self.final_norm.load_params(get)
        self.head.load_params(get, tied_table=getattr(self.embedding, "table", None))

    def weight_bytes(self) -> int:
        seen, total = set(), 0
        stack = [self]
        while stack:
            o = stack.pop()
            for v in (vars(o).values() if hasattr(o, "__dict__") else ()):
                if isinstance(v, torch.Tensor):
                    if v.data_ptr() not in seen:
                        seen.add(v.data_ptr())
                        total += v.numel() * v.element_size()
                elif isinstance(v, (list, tuple)):
                    stack.extend(x for x in v if hasattr(x, "__dict__"))
                elif hasattr(v, "__dict__") and not isinstance(v, (Runtime, ModelSpec, PartSpec, type)):
                    stack.append(v)
        return total

    def batch_needs(self):
        """The index arrays that the parts' kernels want laid out with every step's batch."""
        if self._batch_needs is None:
            from ..parts.base import BatchNeeds
            needs = BatchNeeds()
            for p in (self.embedding, *self.layers, self.final_norm, self.head):
                needs = needs.merged(p.batch_needs())
            self._batch_needs = needs
        return self._batch_needs

    @property
    def graph_safe(self) -> bool:
        return all(p.graph_safe for p in (self.embedding, *self.layers, self.final_norm, self.head))

    # ---- cache ------------------------------------------------------------
    def cache_needs(self) -> Tuple[List[object], List[Optional[int]]]:
        needs = [self.layers[e.layer].cache_need() for e in self.order]
        sources = [e.cache_from for e in self.order]
        return needs, sources

    # ---- forward ----------------------------------------------------------
    def forward(self, ctx, cache) -> Optional[torch.Tensor]:
        """Run the step's tokens through every entry of the order; return the
        float32 logits [wanted, vocab] at the wanted rows (None if none)."""
        h = self.spec.hidden_size
        x = ctx.ws.buffer("model.residual", (ctx.num_tokens, h), torch.float32)
        self.embedding.forward(ctx.ids, x, ctx.id_src, ctx.feedback)
        stream = ResidualStream(x, ctx.ws)
        for i, e in enumerate(self.order):
            # the block is told through which norm the next one reads what it leaves
            follower = self.layers[self.order[i + 1].layer] if i + 1 < len(self.order) else None
            stream.next_norm = follower.first_norm() if follower is not None else None
            self.layers[e.layer].forward(stream, ctx, cache.view(i))
        x = stream.tensor()
        if ctx.num_want == 0:
            return None
        rows = ctx.ws.buffer("model.rows", (ctx.num_want, h), torch.float32)
        ops.gather_rows(x, ctx.want_rows, rows)
        xn = ctx.ws.buffer("model.rows_normed", (ctx.num_want, h), self.rt.dtype)
        self.final_norm.forward(rows, xn)
        logits = torch.empty((ctx.num_want, self.spec.vocab_size), dtype=torch.float32,
                             device=self.rt.device)
        self.head.forward(xn, logits, ctx.ws)
        return logits


def expected_params_of_spec(spec: ModelSpec) -> Dict[str, ParamSpec]:
    """The tensors a checkpoint of this model holds, without building anything
    on a device."""
    return Model(spec, Runtime(torch.device("cpu"), torch.float32)).expected_params()
