"""RMSNorm: y = (x * rsqrt(mean(x^2) + eps)) * w, the weight multiplying directly
(src/minillm/kernels.cpp:209-216).  The residual add that precedes a norm in the layer is
fused into the same kernel."""
from __future__ import annotations

from ..weights.loader import WeightSpec
from .registry import register_part


@register_part("norm", "rmsnorm")
class RmsNorm:
    graph_safe = True        # forward launches kernels over the step's device vectors only
    fusable_rmsnorm = True   # a following projection may do this norm itself (weight, eps as here)
    def __init__(self, spec):
        self.size, self.eps = spec.size, float(spec.eps)
        self.weight = None

    def weight_specs(self):
        return {"weight": WeightSpec((self.size,), keep_float32=True)}

    def bind(self, weights):
        self.weight = weights["weight"]

    def libraries(self):
        return ["elementwise"]

    def forward(self, ctx, h, delta, out, rows=None, write_h=True):
        ctx.kernels.add_rmsnorm(h, delta, self.weight, out, self.eps, rows=rows, write_h=write_h)
        return out
