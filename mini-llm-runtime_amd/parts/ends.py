"""The two ends of a decoder: the embedding that turns a step's token ids into the float residual stream
(src/minillm/runtime.cpp:224-228, src/minillm/cuda/runtime.cpp:184-188) and the output head that turns the
normed rows whose logits are wanted into logits (src/minillm/runtime.cpp:338-351).  Both are parts like any
other: built from a spec by its `kind`, asked for their tensors, their kernel libraries and their scratch
buffers, so that a model with a multiplier on its embedding, a cap on its logits or a bias on its head
registers another kind instead of editing the model."""
from __future__ import annotations

import torch

from ..config.specs import EmbedSpec, HeadSpec
from ..weights.loader import WeightSpec
from .registry import PartError, register_part

__all__ = ["TokenEmbedding", "LinearHead", "EmbedSpec", "HeadSpec"]


@register_part("embed", "token_embedding")
class TokenEmbedding:
    graph_safe = True        # forward launches kernels over the step's device vectors only

    def __init__(self, spec):
        if spec.vocab_size < 1 or spec.hidden < 1:
            raise PartError("an embedding needs a vocabulary and a width")
        self.spec = spec
        self.weight = None

    def weight_specs(self):
        return {"weight": WeightSpec((self.spec.vocab_size, self.spec.hidden))}

    def bind(self, weights):
        self.weight = weights["weight"]

    def libraries(self):
        return ["elementwise"]

    def workspace_plan(self, rows, logits_rows, dtype, limits):
        return {("hidden", torch.float32): rows * self.spec.hidden}

    def table(self):
        """The [vocab, hidden] matrix, for a head that is tied to it."""
        return self.weight

    def forward(self, ctx):
        """The float residual stream [B, E] of the step's tokens."""
        h = ctx.workspace.get("hidden", (ctx.n_tokens, self.spec.hidden), torch.float32)
        ctx.kernels.embed_gather(ctx.token_ids, self.weight, h)
        return h


@register_part("head", "linear_head")
class LinearHead:
    graph_safe = True

    def __init__(self, spec):
        self.spec = spec
        self.weight = None

    def weight_specs(self):
        # (a tied head has no tensor of its own; a file that carries one anyway is taken at its word)
        return {"weight": WeightSpec((self.spec.vocab_size, self.spec.hidden), optional=self.spec.tied)}

    def bind(self, weights, embed=None):
        """`embed`: the model's embedding part; a tied head without a tensor of its own takes its table (the
        same memory, no copy)."""
        if "weight" in weights:
            self.weight = weights["weight"]
        elif self.spec.tied and embed is not None and hasattr(embed, "table"):
            self.weight = embed.table()
        else:
            raise PartError("the output head has no weight and nothing to be tied to")

    def libraries(self):
        return ["gemm"]

    def workspace_plan(self, rows, logits_rows, dtype, limits):
        return {("logits", torch.float32): logits_rows * self.spec.vocab_size}

    def forward(self, ctx, final):
        """float logits [R, V] of the normed rows `final` [R, E]."""
        logits = ctx.workspace.get("logits", (final.shape[0], self.spec.vocab_size), torch.float32)
        ctx.kernels.gemm(final, self.weight, logits)
        return logits
