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
                 page_size=16, split_keys=256, split_max_tokens=256):
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
        self._upload = Uploader(4 * self.max_batch_tokens, self.device)
        self._meta = torch.empty(4 * self.max_batch_tokens, dtype=torch.int32, device=self.device)
        self.poisoned = False
        self.steps = 0

    # -- requests ------------------------------------------------------------------------------
    def open_request(self):
        return self.cache.acquire_slot()

    def close_request(self, slot):
        self.cache.release_slot(slot)

    def length(self, slot):
        return self.cache.length(slot)

    def free_slots(self):
        return self.cache.book.free_slots()

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
        self.cache.prepare(slots, counts)                 # raises, nothing changed
        first = [self.cache.length(s) for s in slots]
        self.cache.commit(slots, counts)
        try:
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
