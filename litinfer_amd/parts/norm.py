"""RMSNorm: y = w * x / sqrt(mean(x^2) + eps), computed in 32-bit
(src/ops/rms_norm/op.cpp:13-23: eps inside the root, the weight multiplies
directly)."""
from __future__ import annotations

from ..kernels import ops
from ..weights.loader import ParamSpec
from .base import Norm, RmsScaling, register_part


class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.size = int(spec.args["size"])
        self.eps = float(spec.args["eps"])
        if self.eps < 0:
            raise ValueError(f"rmsnorm: eps must not be negative, found {self.eps}")
        self.weight = None

    def expected_params(self):
        return {self.prefix + "weight": ParamSpec((self.size,), init="one_plus_normal")}

    def load_params(self, get):
        self.weight = self.rt.vector(get(self.prefix + "weight"))

    def forward(self, x, out):
        ops.rmsnorm(x, self.weight, self.eps, out)
        return out

    def as_scaling(self):
        return RmsScaling(self.weight, self.eps)


register_part("norm", "rmsnorm", RMSNorm)
