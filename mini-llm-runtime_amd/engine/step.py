"""The step function: one batch of (request, its next tokens) -- portions of prompts beside
single decoded tokens, cut anywhere -- run as one batch from the cache, logits returned at the
wanted places only.  This is the engine's counterpart of the reference's `forward` over a flat
batch of input tokens (src/minillm/cuda/runtime.cpp:146-254): validate and reserve without side
effects, commit the pages, upload the metadata in one copy, run the layers, give back what
windows have passed.  Generation, trace replay and the benchmark all go through `Runner.step`.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Sequence

import torch

from ..cache.manager import CacheManager
from ..kernels import Kernels
from .context import StepContext, Uploader, Workspace


class StepError(ValueError):
    """The batch was refused before anything was changed."""


@dataclass
class Entry:
    slot: int
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=list)     # places among `tokens` whose logits are asked for


class Runner:
    def __init__(self, model, max_tokens, max_slots=4, max_length=None, max_batch_tokens=None,
                 page_size=16, split_keys=256, split_max_tokens=256, use_graphs=True, graph_max_batch=256,
                 target_workgroups=512):
        self.model = model
        self.dtype, self.device = model.dtype, model.device
        spec = model.spec
        self.max_length = min(max_length or spec.max_positions, spec.max_positions)
        self.max_batch_tokens = max_batch_tokens or self.max_length
        self.kernels = Kernels(self.dtype)
        self.kernels.prepare(model.libraries())
        self.cache = CacheManager(model.cache_entry_specs, self.dtype, self.device, page_size,
                                  max_tokens, max_slots, self.max_length)
        self.workspace = Workspace(self.device)
        self.ctx = StepContext(self.kernels, self.cache, self.workspace, self.dtype, self.max_length,
                               split_keys, split_max_tokens)
        self.ctx.target_workgroups = target_workgroups
        self._upload = Uploader(4 * self.max_batch_tokens, self.device)
        self._meta = torch.empty(4 * self.max_batch_tokens, dtype=torch.int32, device=self.device)
        self.poisoned = False
        self.steps = 0
        # steps of single tokens (decoding) are launch-bound: after a first eager run a batch size is
        # captured once as a HIP graph over fixed buffers and replayed from then on
        self.use_graphs = use_graphs and model.graph_safe()
        self.graph_max_batch = graph_max_batch
        self._decode_graphs = {}

    # -- requests ------------------------------------------------------------------------------
    def open_request(self):
        return self.cache.acquire_slot()

    def close_request(self, slot):
        self.cache.release_slot(slot)

    def length(self, slot):
        return self.cache.length(slot)

    def free_slots(self):
        return self.cache.book.free_slots()

    # -- decoding steps as graphs --------------------------------------------------------------
    def _decode_step(self, entries, first):
        """One token per request, logits wanted for each: the same kernels as any step, launched from a
        captured graph.  The graph's buffers are fixed: token ids, positions, slots and wanted rows live
        in a vector of their own per batch size, key splits are laid out for the longest context, and the
        logits land in the usual scratch buffer."""
        n = len(entries)
        state = self._decode_graphs.get(n)
        if state is None:
            meta = torch.empty(4 * n + 2 * n, dtype=torch.int32, device=self.device)
            meta[3 * n:4 * n] = torch.arange(n, dtype=torch.int32, device=self.device)      # wanted rows
            meta[4 * n:5 * n] = torch.arange(n, dtype=torch.int32, device=self.device)      # groups: row i ...
            meta[5 * n:6 * n] = 1                                                           # ... one token each
            state = dict(meta=meta, upload=Uploader(3 * n, self.device), graph=None, logits=None, runs=0)
            self._decode_graphs[n] = state
        meta = state["meta"]
        state["upload"].send([int(e.tokens[0]) for e in entries] + list(first) + [e.slot for e in entries], meta)
        if state["graph"] is not None:
            state["graph"].replay()
            return state["logits"]
        ctx = self.ctx
        ctx.begin_step()
        ctx.n_tokens = n
        ctx.token_ids, ctx.positions, ctx.slots = meta[0:n], meta[n:2 * n], meta[2 * n:3 * n]
        ctx.segments = [(e.slot, i, 1, p0) for i, (e, p0) in enumerate(zip(entries, first))]
        ctx.max_context = self.max_length                 # the graph must serve every later context
        ctx.single_token_groups = (meta[4 * n:5 * n], meta[5 * n:6 * n], n)        # groups of one token each
        want_rows = meta[3 * n:4 * n]
        state["runs"] += 1
        if state["runs"] == 1:                            # first time: eager, sizes the scratch buffers
            return self.model.forward(ctx, want_rows)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            logits = self.model.forward(ctx, want_rows)
        state["graph"], state["logits"] = graph, logits
        graph.replay()
        return logits

    # -- the step ------------------------------------------------------------------------------
    def _validate(self, entries):
        if self.poisoned:
            raise StepError("an earlier step failed after it had started; build a new runner")
        if not entries:
            raise StepError("empty batch")
        vocab = self.model.spec.vocab_size
        total = 0
        for e in entries:
            n = len(e.tokens)
            if n == 0:
                raise StepError("a batch entry must bring at least one token")
            total += n
            for t in e.tokens:
                if not 0 <= int(t) < vocab:
                    raise StepError(f"token id {t} is outside the vocabulary [0, {vocab})")
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise StepError(f"wanted place {w} is outside the entry's {n} tokens")
        if total > self.max_batch_tokens:
            raise StepError(f"{total} tokens exceed the step's limit of {self.max_batch_tokens}")
        return total

    def step(self, entries: List[Entry]):
        """Returns float logits [R, V] on the device (R = wanted places, in the order of the
        entries and of their `want`), or None when nothing is wanted."""
        total = self._validate(entries)
        slots = [e.slot for e in entries]
        counts = [len(e.tokens) for e in entries]
        first = self.cache.commit_first(slots, counts)    # raises with nothing changed, else takes the pages
        try:
            if (self.use_graphs and total == len(entries) <= self.graph_max_batch
                    and all(list(e.want) == [0] for e in entries)):
                logits = self._decode_step(entries, first)
                self.cache.retire(slots)
                self.steps += 1
                return logits
            ids, pos, slot_of, rows = [], [], [], []
            segments = []
            for e, p0 in zip(entries, first):
                base = len(ids)
                n = len(e.tokens)
                segments.append((e.slot, base, n, p0))
                ids.extend(int(t) for t in e.tokens)
                pos.extend(range(p0, p0 + n))
                slot_of.extend([e.slot] * n)
                rows.extend(base + int(w) for w in e.want)
            r = len(rows)
            self._upload.send(ids + pos + slot_of + rows, self._meta)
            ctx = self.ctx
            ctx.begin_step()
            ctx.n_tokens = total
            ctx.token_ids = self._meta[0:total]
            ctx.positions = self._meta[total:2 * total]
            ctx.slots = self._meta[2 * total:3 * total]
            ctx.segments = segments
            ctx.max_context = max(p0 + n for (_, _, n, p0) in segments)
            want_rows = self._meta[3 * total:3 * total + r] if r else None
            logits = self.model.forward(ctx, want_rows)
            self.cache.retire(slots)
            self.steps += 1
            return logits
        except Exception:
            self.poisoned = True
            raise
