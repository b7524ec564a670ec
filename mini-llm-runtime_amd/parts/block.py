"""Arrangement of the parts in a layer.  Pre-norm residual block (src/minillm/runtime.cpp:245-337):
h += mixer(norm1(h)); h += ffn(norm2(h)).  The residual stream h is float; every add into it is
fused with the norm that follows, so a block hands its last output on as `pending` instead of
adding it itself."""
from __future__ import annotations

from .registry import Handoff, build_part, register_part


@register_part("block", "prenorm")
class PreNormBlock:
    graph_safe = True        # forward launches kernels over the step's device vectors only
    def __init__(self, spec):
        self.norm1 = build_part("norm", spec.norm1)
        self.mixer = build_part("mixer", spec.mixer)
        self.norm2 = build_part("norm", spec.norm2)
        self.ffn = build_part("ffn", spec.ffn)

    def parts(self):
        return {"norm1": self.norm1, "mixer": self.mixer, "norm2": self.norm2, "ffn": self.ffn}

    def workspace_plan(self, rows, dtype, limits):
        import torch
        width = self.norm1.size
        few = min(rows, 16)
        return {("normed", dtype): rows * width, ("handoff_x", dtype): few * width,
                ("handoff_ss", torch.float32): few * max(1, (width + 15) // 16)}

    def forward(self, ctx, h, pending, cache_id, write_cache=True, next_norm=None):
        fusable = lambda norm: norm is not None and getattr(norm, "fusable_rmsnorm", False) and norm.size == h.shape[1]
        if (ctx.kernels.handoff_supported(h.shape[0]) and fusable(self.norm1) and fusable(self.norm2)
                and hasattr(self.mixer, "forward_handoff") and hasattr(self.ffn, "forward_handoff")):
            # few rows: every norm is shared between the projection before it (which adds into h and leaves
            # h * weight and partial sums of squares) and the projection after it (which applies the scale)
            hand = pending if isinstance(pending, Handoff) and pending.norm is self.norm1 else \
                self.norm1.prenorm(ctx, h, None if isinstance(pending, Handoff) else pending)
            hand = self.mixer.forward_handoff(ctx, hand, h, self.norm2, cache_id, write_cache)
            return self.ffn.forward_handoff(ctx, hand, h, next_norm if fusable(next_norm) else None)
        if isinstance(pending, Handoff):                  # h is complete already
            pending = None
        normed = ctx.workspace.get("normed", tuple(h.shape), ctx.dtype)
        self.norm1.forward(ctx, h, pending, normed)
        mixed = self.mixer.forward(ctx, normed, cache_id, write_cache)
        self.norm2.forward(ctx, h, mixed, normed)
        return self.ffn.forward(ctx, normed)
