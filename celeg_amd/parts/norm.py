"""RMSNorm: y = x / sqrt(mean(x^2) + eps) * w, eps inside the root, w a plain scale
(src/backend/cpu/kernels/elementwise.cpp:56-76; CUDA kernels/norm.cuh:1-44).
The sum of squares and the scaling are done in 32-bit whatever the activation dtype."""
from __future__ import annotations

from .base import Norm, WeightSpec, register_part


class RmsNorm(Norm):
    graph_safe = True

    def __init__(self, spec):
        super().__init__(spec)
        self.width = int(self.params["width"])
        self.eps = float(self.params["eps"])
        if self.width <= 0 or not self.eps > 0:
            raise ValueError("rmsnorm: width and eps must be positive")
        self.weight = None

    def weight_specs(self):
        return {"weight": WeightSpec((self.width,), kind="vector", init="around_one")}

    def load(self, tensors, rt):
        self.weight = tensors["weight"]

    def forward(self, x, out, rt, delta=None, rows=None):
        """out = norm(x [+ delta]).  With ``delta`` and no ``rows`` the sum is written
        back to ``x`` (the residual stream); with ``rows`` only those rows are read and
        ``x`` is left alone."""
        rt.ops.rmsnorm(x, self.weight, self.eps, out, delta=delta, rows=rows)
        return out


register_part("norm", "rmsnorm", RmsNorm)
