"""A decoder model put together from a `ModelSpec`: an embedding part, the layers (blocks of parts) in
the order the schedule gives, a final norm on the wanted rows and an output head part.

Which class builds which part is decided by the specs' `kind`s through the parts registry;
which tensor of the file feeds which part is decided by the architecture's configuration
class (`global_tensor_name`, `layer_tensor_name`).  The model itself knows no architecture.
"""
from __future__ import annotations

from dataclasses import replace

import torch

from ..config import load_config
from ..weights.loader import WeightSpec, load_weights
from .registry import Handoff, PartError, build_part


def build_blocks(spec):
    return [build_part("block", layer) for layer in spec.layers]


def _tensor_plan(config, spec, blocks):
    """([(global name, WeightSpec, owner, local name)] for every tensor of the model, the embedding part, the
    final norm, the head part); owner is ("embed",), ("final_norm",), ("head",) or (layer index, part name)."""
    embed = build_part("embed", spec.embed_spec())
    final = build_part("norm", spec.final_norm)
    head = build_part("head", spec.head_spec())
    plan = []
    for owner, part in (("embed", embed), ("final_norm", final), ("head", head)):
        for local, ws in part.weight_specs().items():
            plan.append((config.global_tensor_name(f"{owner}.{local}"), ws, (owner,), local))
    for i, block in enumerate(blocks):
        for part_name, part in block.parts().items():
            for local, ws in part.weight_specs().items():
                if ws.stack is not None:              # a stack belongs to one part of one layer
                    ws = replace(ws, stack=f"{i}.{part_name}.{ws.stack}")
                plan.append((config.layer_tensor_name(i, part_name, local), ws, (i, part_name), local))
    names = [p[0] for p in plan]
    if len(set(names)) != len(names):
        raise PartError("two parts claim the same tensor name")
    return plan, embed, final, head


def expected_tensors(config):
    """{tensor name: WeightSpec} of the architecture described by `config`."""
    spec = config.model_spec()
    plan = _tensor_plan(config, spec, build_blocks(spec))[0]
    return {name: ws for name, ws, _, _ in plan}


class DecoderModel:
    def __init__(self, config, weights, dtype, device):
        """`weights`: {tensor name: device tensor} as `load_weights` returns them."""
        self.config = config
        self.spec = spec = config.model_spec()
        self.dtype, self.device = dtype, torch.device(device)
        self.arena = None                     # the planned allocation that holds the weights (set by `load`)
        if len(spec.schedule) == 0:
            raise PartError("the schedule runs no layer")
        for run in spec.schedule:
            if not 0 <= run.layer < len(spec.layers):
                raise PartError(f"the schedule names layer {run.layer} of {len(spec.layers)}")
        self.blocks = build_blocks(spec)
        plan, self.embed, self.final_norm, self.head = _tensor_plan(config, spec, self.blocks)
        by_owner = {}
        for name, ws, owner, local in plan:
            if name in weights:
                by_owner.setdefault(owner, {})[local] = weights[name]
        self.embed.bind(by_owner.get(("embed",), {}))
        self.final_norm.bind(by_owner[("final_norm",)])
        self.head.bind(by_owner.get(("head",), {}), embed=self.embed)      # (tied: the embedding's memory, no copy)
        for i, block in enumerate(self.blocks):
            for part_name, part in block.parts().items():
                part.bind(by_owner.get((i, part_name), {}))
        # cache entries: one per cache id the schedule names
        n_entries = 1 + max(run.cache for run in spec.schedule)
        self.cache_entry_specs = [None] * n_entries
        writers = set()
        for run in spec.schedule:
            cs = self.blocks[run.layer].mixer.cache_spec()
            if self.cache_entry_specs[run.cache] is None:
                self.cache_entry_specs[run.cache] = cs
            elif self.cache_entry_specs[run.cache] != cs:
                raise PartError(f"cache entry {run.cache} is shared by mixers with different needs")
            if run.write_cache:
                writers.add(run.cache)
        for cid in range(n_entries):
            if self.cache_entry_specs[cid] is not None and cid not in writers:
                raise PartError(f"cache entry {cid} is read but never written")

    @classmethod
    def load(cls, folder, dtype, device="cuda:0", device_budget_bytes=None):
        """`device_budget_bytes`: None for no gate; else the weights' planned bytes are checked against
        min(this cap (0: none), 80 % of the free device memory, free - 512 MiB) before anything is allocated."""
        config = load_config(folder)
        arena = []
        weights = load_weights(folder, expected_tensors(config), dtype, device, device_budget_bytes, arena)
        model = cls(config, weights, dtype, device)
        model.arena = arena[0]
        return model

    def _ends(self):
        return [self.embed, self.final_norm, self.head]

    def libraries(self):
        """The kernel libraries that the parts of this model launch (each part names its own)."""
        names = set()
        if self.dtype == torch.bfloat16:
            names.add("library_gemm")            # projections of many rows go to the vendor library
        for part in self._ends() + [p for block in self.blocks for p in block.parts().values()]:
            if hasattr(part, "libraries"):
                names.update(part.libraries())
        return sorted(names)

    def workspace_plan(self, rows, logits_rows, limits):
        """{(buffer name, dtype): elements} of every scratch buffer that a step of at most `rows` tokens with
        at most `logits_rows` wanted places asks for: the final norm's rows here, the rest from the parts that
        state theirs (the ends: `workspace_plan(rows, logits_rows, dtype, limits)`; blocks and their parts:
        `workspace_plan(rows, dtype, limits)`; a part without one gets its buffers on demand)."""
        plan = {("final", self.dtype): logits_rows * self.spec.hidden}

        def add(part_plan):
            for key, count in part_plan.items():
                plan[key] = max(plan.get(key, 0), count)
        for part in (self.embed, self.head):
            if hasattr(part, "workspace_plan"):
                add(part.workspace_plan(rows, logits_rows, self.dtype, limits))
        for block in self.blocks:
            for part in [block, *block.parts().values()]:
                if hasattr(part, "workspace_plan"):
                    add(part.workspace_plan(rows, self.dtype, limits))
        return plan

    def graph_safe(self):
        """True when every part of every layer may be captured in a graph."""
        return all(getattr(part, "graph_safe", False) for block in self.blocks
                   for part in [block, *block.parts().values()]) and all(getattr(part, "graph_safe", False)
                                                                         for part in self._ends())

    def weight_bytes(self):
        """Bytes of the tensors the model uses (each once; without the padding between them)."""
        seen, total = set(), 0
        tensors = []
        for part in self._ends() + [p for block in self.blocks for p in block.parts().values()]:
            tensors += [v for v in vars(part).values() if isinstance(v, torch.Tensor)]
        for t in tensors:
            if t.data_ptr() not in seen:
                seen.add(t.data_ptr())
                total += t.numel() * t.element_size()
        return total

    def forward(self, ctx, want_rows):
        """Run the step's tokens through every scheduled layer; logits float [R, V] at the rows
        `want_rows` (device int32, indices into the step's tokens), or None when R = 0."""
        k = ctx.kernels
        status = getattr(ctx, "status", None)            # the debug mode that looks at the hidden state
        if status is not None:
            k.status_reset(status)
        h = self.embed.forward(ctx)
        pending = None
        schedule = self.spec.schedule
        for i, run in enumerate(schedule):
            # (the norm the next run starts with: a block may prepare it while it adds its last output into h)
            next_norm = self.blocks[schedule[i + 1].layer].norm1 if i + 1 < len(schedule) else None
            pending = self.blocks[run.layer].forward(ctx, h, pending, run.cache, run.write_cache, next_norm=next_norm)
            if isinstance(pending, Handoff) and i + 1 == len(schedule):
                pending = None                            # (h is complete)
            if status is not None:                        # h + pending is the hidden state after this run
                k.finite_check(h, None if isinstance(pending, Handoff) else pending, i, status)
        if ctx.cache is not None and ctx.cache.has_state():
            ctx.cache.commit_state(ctx.segment_slots)     # every layer has run: the staged state becomes live
        r = 0 if want_rows is None else want_rows.numel()
        if r == 0:
            return None
        final = ctx.workspace.get("final", (r, self.spec.hidden), self.dtype)
        self.final_norm.forward(ctx, h, pending, final, rows=want_rows, write_h=False)
        return self.head.forward(ctx, final)
