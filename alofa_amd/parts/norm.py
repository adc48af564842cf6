"""RMSNorm: y = x / sqrt(mean(x^2) + eps) * w; the weight multiplies after the
scale, eps sits inside the root, no 1+w, no bias
(src/alofa/kernels/cpu/scalar.mojo:93-129)."""
from __future__ import annotations

from .. import ops
from ..weights.loader import TensorRule
from .base import Norm, register_part


class RMSNorm(Norm):
    """params: name (tensor name), width, eps."""

    @classmethod
    def tensors(cls, spec):
        return {spec.params["name"]: TensorRule((spec.params["width"],), "norm")}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.eps = float(spec.params["eps"])
        self.width = int(spec.params["width"])
        self.weight = rt.vector(weights[spec.params["name"]])

    def as_rmsnorm(self):
        return self.weight, self.eps

    def forward(self, out, x, rows=None):
        ops.rmsnorm(out, x, self.weight, self.eps, self.rt.exact, rows)


register_part("norm", "rmsnorm", RMSNorm)
