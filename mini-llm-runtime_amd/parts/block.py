"""Arrangement of the parts in a layer.  Pre-norm residual block (src/minillm/runtime.cpp:245-337):
h += mixer(norm1(h)); h += ffn(norm2(h)).  The residual stream h is float; every add into it is
fused with the norm that follows, so a block hands its last output on as `pending` instead of
adding it itself."""
from __future__ import annotations

from .registry import build_part, register_part


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
        return {("hidden_alt", torch.float32): min(rows, 16) * width, ("normed", dtype): rows * width}

    def forward(self, ctx, h, pending, cache_id, write_cache=True):
        if (ctx.kernels.norm_gemm_supported(h.shape[0], h.shape[1])
                and getattr(self.norm1, "fusable_rmsnorm", False) and getattr(self.norm2, "fusable_rmsnorm", False)
                and hasattr(self.mixer, "forward_prenorm") and hasattr(self.ffn, "forward_prenorm")):
            # few rows: each norm rides in the projection that follows it; the residual stream goes to a
            # second buffer and back, so that no workgroup reads a row that another one is updating
            h_alt = ctx.workspace.get("hidden_alt", tuple(h.shape), h.dtype)
            mixed = self.mixer.forward_prenorm(ctx, h, pending, self.norm1, h_alt, cache_id, write_cache)
            return self.ffn.forward_prenorm(ctx, h_alt, mixed, self.norm2, h)
        normed = ctx.workspace.get("normed", tuple(h.shape), ctx.dtype)
        self.norm1.forward(ctx, h, pending, normed)
        mixed = self.mixer.forward(ctx, normed, cache_id, write_cache)
        self.norm2.forward(ctx, h, mixed, normed)
        return self.ffn.forward(ctx, normed)
