"""SwiGLU feed-forward: out = (silu(x Wgate^T) * (x Wup^T)) Wdown^T with silu(g) = g / (1 + exp(-g))
(src/minillm/runtime.cpp:323-336).  Gate and up are one stacked projection."""
from __future__ import annotations

import torch

from ..weights.loader import WeightSpec, stacked
from .registry import Handoff, PartError, register_part


@register_part("ffn", "swiglu")
class SwiGluMlp:
    graph_safe = True        # forward launches kernels over the step's device vectors only
    def __init__(self, spec):
        if spec.activation != "silu":
            raise PartError(f"activation {spec.activation!r} is not built (silu)")
        self.spec = spec
        self.gate_up = None
        self.down = None

    def weight_specs(self):
        s = self.spec
        return {"gate_proj": WeightSpec((s.intermediate, s.hidden), stack="gate_up"),
                "up_proj": WeightSpec((s.intermediate, s.hidden), stack="gate_up"),
                "down_proj": WeightSpec((s.hidden, s.intermediate))}

    def bind(self, weights):
        self.gate_up = stacked([weights["gate_proj"], weights["up_proj"]])
        self.down = weights["down_proj"]

    def libraries(self):
        return ["gemm", "elementwise"]

    def workspace_plan(self, rows, dtype, limits):
        s = self.spec
        return {("act", dtype): rows * s.intermediate, ("gate_up", dtype): rows * 2 * s.intermediate,
                ("ffn_out", dtype): rows * s.hidden}

    def forward_handoff(self, ctx, hand, h, norm_after):
        """As `forward` on the norm that `hand` describes, its scale applied inside the first projection; the
        second projection adds into h and prepares `norm_after` (None: nothing follows)."""
        s = self.spec
        m = h.shape[0]
        k = ctx.kernels
        act = ctx.workspace.get("act", (m, s.intermediate), ctx.dtype)
        k.gemm_prenormed(hand.x, hand.ss, hand.norm.eps, self.gate_up, act, gated=True)
        if norm_after is None:
            k.gemm_residual(act, self.down, h)
            return None
        x = ctx.workspace.get("handoff_x", (m, s.hidden), ctx.dtype)
        ss = ctx.workspace.get("handoff_ss", (m, k.handoff_parts(s.hidden)), torch.float32)
        k.gemm_residual(act, self.down, h, norm_after.weight, x, ss)
        return Handoff(norm_after, x, ss)

    def forward(self, ctx, x):
        s = self.spec
        m = x.shape[0]
        act = ctx.workspace.get("act", (m, s.intermediate), x.dtype)
        if ctx.kernels.gated_silu_fused(m, s.hidden):  # few rows: the activation rides on the projection
            ctx.kernels.gemm_gated_silu(x, self.gate_up, act)
        else:
            gate_up = ctx.workspace.get("gate_up", (m, 2 * s.intermediate), x.dtype)
            ctx.kernels.gemm(x, self.gate_up, gate_up)
            ctx.kernels.silu_mul(gate_up, act)
        out = ctx.workspace.get("ffn_out", (m, s.hidden), x.dtype)
        ctx.kernels.gemm(act, self.down, out)
        return out
