"""RMSNorm: y = (x * rsqrt(mean(x^2) + eps)) * w, the weight multiplying directly
(src/minillm/kernels.cpp:209-216).  The residual add that precedes a norm in the layer is
fused into the same kernel."""
from __future__ import annotations

import torch

from ..weights.loader import WeightSpec
from .registry import register_part


@register_part("norm", "rmsnorm")
class RmsNorm:
    graph_safe = True        # forward launches kernels over the step's device vectors only
    fusable_rmsnorm = True   # the projections before and after it may share this norm between them (weight, eps as here)
    def __init__(self, spec):
        self.size, self.eps = spec.size, float(spec.eps)
        self.weight = None

    def weight_specs(self):
        return {"weight": WeightSpec((self.size,), keep_float32=True)}

    def bind(self, weights):
        self.weight = weights["weight"]

    def libraries(self):
        return ["elementwise"]

    def prenorm(self, ctx, h, delta):
        """h += delta (delta may be None) and the first half of this norm for the projection that follows:
        a `Handoff` (see parts/registry.py)."""
        from .registry import Handoff
        m = h.shape[0]
        x = ctx.workspace.get("handoff_x", (m, self.size), ctx.dtype)
        ss = ctx.workspace.get("handoff_ss", (m, 1), torch.float32)
        ctx.kernels.rows_prenorm(h, delta, self.weight, x, ss)
        return Handoff(self, x, ss)

    def forward(self, ctx, h, delta, out, rows=None, write_h=True):
        ctx.kernels.add_rmsnorm(h, delta, self.weight, out, self.eps, rows=rows, write_h=write_h)
        return out
