"""Dense SwiGLU feed-forward: down(silu(gate(x)) * up(x)), no biases; silu is
x / (1 + exp(-x)) (src/alofa/kernels/cpu/scalar.mojo:219-231,
src/alofa/engine/executor.mojo:806-837). Gate and up run as one kernel that
applies the activation before anything is written."""
from __future__ import annotations

from .. import ops
from ..weights.loader import TensorRule
from .base import FeedForward, register_part


class SwiGLU(FeedForward):
    """params: prefix, hidden, intermediate."""
    capturable = True   # native kernels on the current stream only: a decode step may be graph-captured

    @classmethod
    def tensors(cls, spec):
        p = spec.params
        pre, h, i = p["prefix"], p["hidden"], p["intermediate"]
        return {pre + "gate_proj.weight": TensorRule((i, h)), pre + "up_proj.weight": TensorRule((i, h)),
                pre + "down_proj.weight": TensorRule((h, i))}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.hidden, self.intermediate = int(p["hidden"]), int(p["intermediate"])
        pre = p["prefix"]
        gate, up = weights[pre + "gate_proj.weight"], weights[pre + "up_proj.weight"]
        if gate.dtype is not up.dtype:
            gate, up = gate.float(), up.float()
        self.w_gate, self.w_up = rt.matrix(gate), rt.matrix(up)
        self.w_down = rt.matrix(weights[pre + "down_proj.weight"])

    def fuses_norm(self, norm, rows):
        return (not self.rt.exact and norm.as_rmsnorm() is not None
                and ops.can_fuse_norm(rows, self.w_gate, self.rt.dtype, swiglu=True))

    gives_normed = True

    def forward(self, ctx, x, residual, norm=None, then=None):
        act = ctx.scratch("ff_act", (residual.shape[0], self.intermediate), self.rt.dtype)
        if norm is not None:      # the norm before the feed-forward rides on the gate/up product
            ops.gemm_swiglu(act, residual, self.w_gate, self.w_up, norm=norm.as_rmsnorm())
        else:
            ops.gemm_swiglu(act, x, self.w_gate, self.w_up, exact=self.rt.exact)
        then_norm = None
        if then is not None:      # the norm behind this part, left in the rows given with it
            weight, eps = then[0].as_rmsnorm()
            then_norm = (weight, eps, then[1])
        ops.gemm(residual, act, self.w_down, add_to_out=True, exact=self.rt.exact, then_norm=then_norm)


register_part("feed_forward", "swiglu", SwiGLU)
