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

import numpy as np
import torch

from ..cache.manager import CacheManager
from ..kernels import Kernels
from ..kernels.ops import LIBRARY_GEMM_WORKSPACE
from ..kernels.profile import Profiler
from .context import StepContext, Uploader, Workspace
from .memory import MemoryBudgetError, MemoryPlan, device_budget


class StepError(ValueError):
    """The batch was refused before anything was changed."""


class NonFiniteHidden(RuntimeError):
    """The hidden state held a NaN or an infinity after some layer (check_finite); the runner is poisoned."""


@dataclass
class Entry:
    slot: int
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=list)     # places among `tokens` whose logits are asked for


def _kv_dtype(name, engine_dtype):
    if name in (None, "auto") or name == engine_dtype:
        return engine_dtype
    names = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
             "f32": torch.float32}
    if name in names:
        return names[name]
    raise ValueError(f"kv_dtype must be auto, bfloat16 or float32, got {name!r}")


class Runner:
    def __init__(self, model, max_tokens=None, max_slots=4, max_length=None, max_batch_tokens=None,
                 page_size=16, split_keys=256, split_max_tokens=256, use_graphs=True, graph_max_batch=256,
                 target_workgroups=512, graph_max_tokens=512, graph_after=4, max_graphs=128, library_gemm=True,
                 max_logits_rows=None, device_budget_bytes=None, check_finite=False, profile=False, kv_dtype="auto"):
        """`max_tokens`: tokens the page pool holds, or None: as many as the device's budget leaves room for
        beside everything else that is planned, at most what `max_slots` requests of `max_length` tokens hold
        (the budget is then the rule below also with `device_budget_bytes` None); `max_length`: longest request;
        `max_batch_tokens`: most tokens of one step; `max_logits_rows`: most wanted places of one step (default:
        every token).  `kv_dtype`: the cache's element type, "auto" or the engine's own (the attention kernels
        read the pages as the engine's element type; another one is refused).
        `device_budget_bytes`: None for no gate, else the device memory that the runner will hold is planned and
        compared with min(this cap (0: none), 80 % of the free memory, free - 512 MiB) before the cache is
        allocated (`MemoryBudgetError`).  `check_finite`: after every layer one small kernel looks at the
        hidden state; a NaN or an infinity ends the step with `NonFiniteHidden` naming the first layer and
        row, and poisons the runner (one more synchronisation a step: a debug mode).  `profile`: events
        around every launch, summed per kernel class (`profile_report`); steps then run eagerly."""
        self.model = model
        self.dtype, self.device = model.dtype, model.device
        spec = model.spec
        self.max_length = min(max_length or spec.max_positions, spec.max_positions)
        self.max_batch_tokens = max_batch_tokens or self.max_length
        # library_gemm=False: every product on the hand-written kernels (the vendor library takes none)
        self.kernels = Kernels(self.dtype, library_gemm=library_gemm)
        self.kernels.prepare(model.libraries())
        for block in model.blocks:                        # sizes that no step could serve are refused now
            for part in block.parts().values():
                if hasattr(part, "check_limits"):
                    part.check_limits(self.kernels, self.max_length, page_size, split_keys)
        self.max_logits_rows = min(max_logits_rows or self.max_batch_tokens, self.max_batch_tokens)
        # the memory plan, and the budget gate before anything of it is allocated
        limits = dict(max_length=self.max_length, page_size=page_size, split_keys=split_keys,
                      split_max_tokens=split_max_tokens, target_workgroups=target_workgroups)
        workspace_plan = model.workspace_plan(self.max_batch_tokens, self.max_logits_rows, limits)
        uses_library = library_gemm and self.dtype == torch.bfloat16
        if _kv_dtype(kv_dtype, self.dtype) != self.dtype:
            raise ValueError(f"kv_dtype {kv_dtype}: the {self.dtype} engine's attention kernels read pages of their own "
                             "element type only")
        if max_tokens is None:
            # the pool takes what the budget leaves beside the scratch buffers, the metadata and the library's
            # scratch (the weights are resident already and no longer part of the free memory)
            other = MemoryPlan(workspace=Workspace.plan_bytes(workspace_plan), metadata=5 * 4 * self.max_batch_tokens + 8,
                               library_scratch=LIBRARY_GEMM_WORKSPACE if uses_library else 0).to_allocate()
            room = device_budget(device_budget_bytes or 0, self.device) - other
            max_tokens = CacheManager.tokens_that_fit(model.cache_entry_specs, self.dtype, page_size, max_slots,
                                                      self.max_length, room)
            if max_tokens <= 0:
                raise MemoryBudgetError(f"the device's budget leaves {room} bytes for the cache: not one page a group")
            if device_budget_bytes is None:
                device_budget_bytes = 0
        self.max_tokens = max_tokens
        kv, tables, state = CacheManager.plan(model.cache_entry_specs, self.dtype, page_size, max_tokens, max_slots,
                                              self.max_length)
        self.memory_plan = MemoryPlan(
            weights=model.arena.planned if model.arena is not None else model.weight_bytes(),
            kv_pages=kv, block_tables=tables, state=state, workspace=Workspace.plan_bytes(workspace_plan),
            metadata=5 * 4 * self.max_batch_tokens + 8, library_scratch=LIBRARY_GEMM_WORKSPACE if uses_library else 0)
        self.memory_plan.check(device_budget_bytes, self.device)
        self.cache = CacheManager(model.cache_entry_specs, self.dtype, self.device, page_size,
                                  max_tokens, max_slots, self.max_length)
        assert (self.cache.kv_bytes(), self.cache.table_bytes(), self.cache.state_bytes()) == (kv, tables, state), \
            "the cache holds other sizes than were planned"
        self.workspace = Workspace(self.device)
        self.workspace.reserve(workspace_plan)
        if uses_library:
            self.kernels.reserve_library_workspace(self.device)
        self.check_finite = bool(check_finite)
        self._status = torch.zeros(2, dtype=torch.int32, device=self.device)
        if profile:
            self.kernels.profiler = Profiler()
            use_graphs = False                            # events inside a captured graph measure nothing
        self.ctx = StepContext(self.kernels, self.cache, self.workspace, self.dtype, self.max_length,
                               split_keys, split_max_tokens)
        self.ctx.target_workgroups = target_workgroups
        # split attention keeps its partial results within what was planned for them
        self.ctx.partial_budget = workspace_plan.get(("attn_partial", torch.float32))
        self.ctx.status = self._status if self.check_finite else None
        # one vector a step: token ids, positions, slots (a value a token), wanted rows, and -- for a model that
        # keeps state per request -- one slot per entry
        self._upload = Uploader(5 * self.max_batch_tokens, self.device)
        self._meta = torch.empty(5 * self.max_batch_tokens, dtype=torch.int32, device=self.device)
        self.poisoned = False
        self.steps = 0
        # steps of few tokens are launch-bound: after a first eager run a step's shape is captured once
        # as a HIP graph over fixed buffers and replayed from then on
        self.use_graphs = use_graphs and model.graph_safe()
        self.graph_max_batch = graph_max_batch            # single tokens in a captured step, at most
        self.graph_max_tokens = max(graph_max_tokens, graph_max_batch)     # tokens in a captured step, at most
        self.graph_after = graph_after                    # a mixed shape is captured after it came this often
        self.max_graphs = max_graphs                      # captured shapes kept (least recently used goes)
        self._graphs = {}
        self._seen = {}
        self.graph_failures = 0                           # shapes whose replays did not match the eager run

    # -- requests ------------------------------------------------------------------------------
    def open_request(self):
        return self.cache.acquire_slot()

    def close_request(self, slot):
        self.cache.release_slot(slot)

    def length(self, slot):
        return self.cache.length(slot)

    def free_slots(self):
        return self.cache.book.free_slots()

    def reserve_unit(self):
        """Tokens in which a scheduler sets a request's pages aside (see `CacheManager.reserve_unit`)."""
        return self.cache.reserve_unit()

    # -- steps as graphs -----------------------------------------------------------------------
    def _signature(self, entries):
        """What a captured step is fixed to: how many tokens every entry brings and where it wants logits."""
        return tuple((len(e.tokens), tuple(int(w) for w in e.want)) for e in entries)

    def _decode_fill(self, entries):
        """(rows of the scratch request, where they go) that fill the single tokens of a batch (each wanting
        its logits) up to a number that comes again: every number up to 8, even ones up to 16, multiples of 4
        up to 64, of 8 beyond.  So that a server whose requests come and go captures a few dozen graphs, not
        one for every number of live requests.  A batch of single tokens only gets the rows at its end; a
        batch whose single tokens come first and prompt portions after them (the scheduler's mixed batches)
        gets them in front, so that the wanted logits stay one block of rows."""
        if self.cache.scratch_slot is None or not self.use_graphs:
            return 0, False
        n = 0
        while n < len(entries) and len(entries[n].tokens) == 1 and list(entries[n].want) == [0]:
            n += 1
        mixed = n < len(entries)
        if n == 0 or (mixed and any(len(e.tokens) == 1 for e in entries[n:])):
            return 0, False
        step = 1 if n <= 8 else 2 if n <= 16 else 4 if n <= 64 else 8
        fill = -(-n // step) * step - n
        total = sum(len(e.tokens) for e in entries) + fill
        wanted = sum(len(e.want) for e in entries) + fill       # (the scratch rows' logits are computed and dropped)
        if (n + fill > self.graph_max_batch or total > min(self.graph_max_tokens, self.max_batch_tokens)
                or wanted > self.max_logits_rows):
            return 0, False
        return fill, mixed

    def _context_bucket(self, longest):
        """The context length a captured step is laid out for: the smallest of 512, 1024, 2048, ... that holds
        the step's longest context (at most max_length).  A graph fixes how many workgroups split a token's
        keys; laid out for max_length, a server with a long limit would launch splits for keys that do not
        exist on every short-context step.  A shape is captured once per bucket it is met in."""
        bucket = 512
        while bucket < longest:
            bucket *= 2
        return min(bucket, self.max_length)

    def _graph_wanted(self, entries, total, sig):
        """Steps are launch-bound unless they bring many tokens.  Steps of single tokens with logits for
        each (decoding) are captured the second time they come, others (portions beside decoded tokens)
        once their shape has come `graph_after` times: a prompt's last portion rarely comes again."""
        if not self.use_graphs or total > self.graph_max_tokens:
            return False
        if sig in self._graphs:
            return True
        shape = sig[0]
        if total == len(shape) and all(w == (0,) for _, w in shape):
            return total <= self.graph_max_batch
        seen = self._seen.get(sig, 0) + 1
        self._seen[sig] = seen
        if len(self._seen) > 4096:
            self._seen.clear()
        return seen > self.graph_after

    @staticmethod
    def _replays_match(graph, result, expect, rewind=lambda: None):
        """Replays the fresh capture twice on the inputs of the eager run that gave `expect`; `result` is
        the tensor that the graph writes.  `rewind` is called before each replay (it puts per-request state
        back to where the step found it)."""
        scale = max(float(expect.abs().nan_to_num(0.0).max()), 1e-30)
        for _ in range(2):
            rewind()
            graph.replay()
            if bool(torch.isfinite(result).all()) != bool(torch.isfinite(expect).all()):
                return False
            if float((result - expect).abs().nan_to_num(0.0).max()) > 1e-3 * scale:
                return False
        return True

    def _graph_step(self, entries, arrays, first, total, sig, fill=0, fill_first=False):
        """The same kernels as any step, launched from a captured graph.  The graph's buffers are fixed:
        token ids, positions and slots live in a vector of their own per shape (the wanted rows and the
        token groups, which depend on the shape only, are written there once), key splits are laid out
        for the longest context, and the logits land in the scratch buffer of the capture.  A shape's
        first run is eager (it sizes the scratch buffers), the second is captured; the capture is then
        replayed twice on the same inputs and compared with the eager result, and a shape whose replays
        differ (a library call that records a clearing node would do that) stays eager for good."""
        state = self._graphs.get(sig)
        shape, bucket = sig
        if state is None:
            rows, base = [], 0
            for n, want in shape:
                rows.extend(base + w for w in want)
                base += n
            # ids | positions | slots | one slot per entry (these change from step to step) | wanted rows (fixed)
            n_seg = len(shape)
            meta = torch.empty(3 * total + n_seg + max(len(rows), 1), dtype=torch.int32, device=self.device)
            if rows:
                meta[3 * total + n_seg:3 * total + n_seg + len(rows)] = torch.tensor(rows, dtype=torch.int32,
                                                                                      device=self.device)
            state = dict(meta=meta, upload=Uploader(3 * total + n_seg, self.device), graph=None, logits=None, runs=0,
                         rows=len(rows), groups={}, keep=None, eager=False)
            self._graphs[sig] = state
            while len(self._graphs) > self.max_graphs:
                self._graphs.pop(next(iter(self._graphs)))
        else:
            self._graphs[sig] = self._graphs.pop(sig)        # most recently used last
        meta = state["meta"]
        rows_of, segments = self._rows(entries, arrays, first, fill, fill_first)
        n_seg = len(segments)
        state["upload"].send(np.concatenate([rows_of.ravel(), np.fromiter((seg[0] for seg in segments), np.int32, n_seg)]),
                             meta)
        if state["graph"] is not None:
            state["graph"].replay()
            return state["logits"]
        ctx = self.ctx
        ctx.begin_step()
        ctx.n_tokens = total
        ctx.token_ids, ctx.positions, ctx.slots = meta[0:total], meta[total:2 * total], meta[2 * total:3 * total]
        ctx.segment_slots = meta[3 * total:3 * total + n_seg]
        ctx.segments = segments
        ctx.single_tokens = total == len(segments)
        r = state["rows"]
        want_rows = meta[3 * total + n_seg:3 * total + n_seg + r] if r else None
        if state["eager"]:                                # a shape whose capture did not hold
            ctx.max_context = max(p0 + n for (_, _, n, p0) in segments)
            return self.model.forward(ctx, want_rows)
        ctx.max_context = bucket                          # the graph must serve every context of its bucket
        ctx.fixed_groups = state["groups"]
        state["runs"] += 1
        if state["runs"] == 1:                            # first time: eager, sizes the scratch buffers
            return self.model.forward(ctx, want_rows)
        # The capture runs the step more than once: eagerly (the reference), then twice as a replay of the
        # fresh graph.  Running a step again writes the same keys and values into the same pages; state of
        # fixed size, which a step ADVANCES, is put back to where the step found it before every further run,
        # so that it has advanced exactly once when this returns.
        before = self.cache.snapshot_state()
        reference = self.model.forward(ctx, want_rows)
        probe = reference if reference is not None else self.workspace.get("hidden", (total, self.model.spec.hidden),
                                                                           torch.float32)
        expect = probe.clone()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            logits = self.model.forward(ctx, want_rows)
        state["keep"] = self.workspace.buffers()
        ok = self._replays_match(graph, logits if logits is not None else probe, expect,
                                 lambda: self.cache.restore_state(before))
        if not ok:
            state["eager"], state["keep"] = True, None
            self.graph_failures += 1
            ctx.fixed_groups = None
            ctx.begin_step()
            ctx.segment_slots = meta[3 * total:3 * total + n_seg]
            ctx.max_context = max(p0 + n for (_, _, n, p0) in segments)
            self.cache.restore_state(before)
            return self.model.forward(ctx, want_rows)
        state["graph"], state["logits"] = graph, logits
        return logits

    def warm_up(self, batch_sizes=None, contexts=None):
        """Captures the decoding steps a server will meet before it meets them, so that no request waits for a
        capture (about 20 ms a shape): for every number of single tokens that `_decode_fill` fills a batch up
        to (at most `max_slots`, or those of `batch_sizes`) and every context bucket (512, 1024, ... up to
        max_length, or those of `contexts`) whose requests fit the page pool, that many requests are opened at
        a context of the bucket, stepped three times (eager, captured, replayed) and closed.  Their pages hold
        zeros meanwhile and are filled with NaN again afterwards.  Short contexts come first, and it stops when
        the runner holds `max_graphs` shapes (one more would push the oldest out again).  To be called while no
        request is open.  Returns the number of graphs captured."""
        if not self.use_graphs or self.poisoned:
            return 0
        if self.free_slots() != self.cache.max_slots:
            raise StepError("warm_up: close every request first")
        limit = min(self.cache.max_slots, self.graph_max_batch)
        if batch_sizes is None:
            batch_sizes = [n for n in range(1, limit + 1)
                           if n % (1 if n <= 8 else 2 if n <= 16 else 4 if n <= 64 else 8) == 0]
        if contexts is None:
            contexts, bucket = [], 512
            while True:
                contexts.append(min(bucket, self.max_length))
                if bucket >= self.max_length:
                    break
                bucket *= 2
        tensors = [t for t in self.cache.paged_tensors() if t.dtype.is_floating_point]
        for t in tensors:
            t.zero_()
        before = sum(1 for st in self._graphs.values() if st["graph"] is not None)
        try:
            for context in contexts:
                bucket = self._context_bucket(context)
                # the first context of the bucket: one beyond the bucket below it (the largest of 512, 1024, ...
                # under this one, which a capped top bucket is not twice of); three steps must stay inside
                below = 512
                while below * 2 < bucket:
                    below *= 2
                start = max(1, min(below + 1, bucket - 4)) if bucket > 512 else 1
                for n in sorted(set(int(b) for b in batch_sizes if 1 <= b <= limit), reverse=True):
                    key = (((1, (0,)),) * n, bucket)
                    if key in self._graphs and self._graphs[key]["graph"] is not None:
                        continue
                    if key not in self._graphs and len(self._graphs) >= self.max_graphs:
                        break
                    if any(n * -(-(start + 4) // size) > pages for size, pages in zip(self.cache.group_page_size,
                                                                                         self.cache.group_pages)):
                        continue                          # that many requests of that length do not fit the pool
                    slots = [self.open_request() for _ in range(n)]
                    try:
                        if start > 1:
                            self.cache.commit(slots, [start - 1] * n)      # (their keys and values: the zeros)
                        for _ in range(3):
                            self.step([Entry(slot, [0], [0]) for slot in slots])
                    finally:
                        for slot in slots:
                            self.close_request(slot)
        finally:
            for t in tensors:
                t.fill_(float("nan"))
        return sum(1 for st in self._graphs.values() if st["graph"] is not None) - before

    # -- the step ------------------------------------------------------------------------------
    def _validate(self, entries):
        if self.poisoned:
            raise StepError("an earlier step failed after it had started; build a new runner")
        if not entries:
            raise StepError("empty batch")
        vocab = self.model.spec.vocab_size
        total = 0
        arrays, wanted = [], []
        for e in entries:
            n = len(e.tokens)
            if n == 0:
                raise StepError("a batch entry must bring at least one token")
            total += n
            arrays.append(self._token_ids(e.tokens, vocab))
            places = len(e.want)
            if places <= 16:                              # (few places: plain comparisons cost less than vectors)
                for w in e.want:
                    if not 0 <= int(w) < n:
                        raise StepError(f"wanted place {w} is outside the entry's {n} tokens")
                if places > 1 and len(set(int(w) for w in e.want)) != places:
                    raise StepError("a wanted place is named twice in one entry")
                want = [int(w) for w in e.want]
            else:
                want = np.asarray(e.want, dtype=np.int64).reshape(-1)
                if want.min() < 0 or want.max() >= n:
                    bad = want[(want < 0) | (want >= n)][0]
                    raise StepError(f"wanted place {bad} is outside the entry's {n} tokens")
                if np.unique(want).size != want.size:
                    # (a place named once bounds the wanted rows by the step's tokens, which the metadata
                    # vector is sized for)
                    raise StepError("a wanted place is named twice in one entry")
            wanted.append(want)
        if total > self.max_batch_tokens:
            raise StepError(f"{total} tokens exceed the step's limit of {self.max_batch_tokens}")
        rows = sum(len(w) for w in wanted)
        if rows > self.max_logits_rows:
            raise StepError(f"{rows} wanted places exceed the step's limit of {self.max_logits_rows}")
        return total, arrays, wanted

    @staticmethod
    def _token_ids(tokens, vocab):
        """An entry's tokens, checked (as they came when they are few, else as an int32 vector); refused when they
        are no whole numbers of the vocabulary."""
        if len(tokens) <= 16:                             # (few tokens: plain comparisons cost less than vectors)
            for t in tokens:
                try:
                    inside = 0 <= t < vocab and int(t) == t
                except (TypeError, ValueError):
                    raise StepError("token ids must be whole numbers") from None
                if not inside:
                    raise StepError(f"token id {t} is outside the vocabulary [0, {vocab})" if isinstance(t, (int, np.integer))
                                    else "token ids must be whole numbers")
            return tokens                                 # (as they came: `_rows` puts them into its vector)
        ids = np.asarray(tokens)
        if ids.ndim != 1 or ids.dtype.kind not in "iub":
            try:                                          # (numbers too large for a machine word, or no numbers)
                ids = np.asarray([int(t) for t in tokens], dtype=object)
            except (TypeError, ValueError):
                raise StepError("token ids must be whole numbers") from None
            if any(t != u for t, u in zip(ids, tokens)):
                raise StepError("token ids must be whole numbers")
        outside = (ids < 0) | (ids >= vocab)
        if outside.any():
            raise StepError(f"token id {ids[outside][0]} is outside the vocabulary [0, {vocab})")
        return ids.astype(np.int32)

    def _rows(self, entries, arrays, first, fill=0, fill_first=False):
        """(token ids | positions | slots of the step's rows as int32 [3, rows], the segments (slot, first row,
        tokens, first position)); `fill` rows of the scratch request (token 0 at position 0) in front or behind."""
        total = sum(len(a) for a in arrays) + fill
        scratch = self.cache.scratch_slot
        if total <= 4 * (len(entries) + fill):
            # mostly single tokens (a decoding step): three short lists and one conversion cost less than
            # a few vector operations for every entry
            ids, pos, slot_of, segments = [], [], [], []
            if fill and fill_first:
                segments = [(scratch, i, 1, 0) for i in range(fill)]
                ids, pos, slot_of = [0] * fill, [0] * fill, [scratch] * fill
            for e, tokens, p0 in zip(entries, arrays, first):
                n = len(tokens)
                segments.append((e.slot, len(ids), n, p0))
                ids.extend(tokens)
                pos.extend(range(p0, p0 + n))
                slot_of.extend([e.slot] * n)
            if fill and not fill_first:
                segments += [(scratch, len(ids) + i, 1, 0) for i in range(fill)]
                ids, pos, slot_of = ids + [0] * fill, pos + [0] * fill, slot_of + [scratch] * fill
            return np.array([ids, pos, slot_of], dtype=np.int32), segments
        rows = np.empty((3, total), dtype=np.int32)
        segments, at = [], 0
        if fill and fill_first:
            rows[0:2, :fill], rows[2, :fill] = 0, scratch
            segments += [(scratch, i, 1, 0) for i in range(fill)]
            at = fill
        for e, ids, p0 in zip(entries, arrays, first):
            n = len(ids)
            rows[0, at:at + n] = ids
            rows[1, at:at + n] = np.arange(p0, p0 + n, dtype=np.int32)
            rows[2, at:at + n] = e.slot
            segments.append((e.slot, at, n, p0))
            at += n
        if fill and not fill_first:
            rows[0:2, at:], rows[2, at:] = 0, scratch
            segments += [(scratch, at + i, 1, 0) for i in range(fill)]
        return rows, segments

    def step(self, entries: List[Entry]):
        """Returns float logits [R, V] on the device (R = wanted places, in the order of the
        entries and of their `want`), or None when nothing is wanted."""
        total, arrays, wanted = self._validate(entries)
        slots = [e.slot for e in entries]
        counts = [len(e.tokens) for e in entries]
        first = self.cache.commit_first(slots, counts)    # raises with nothing changed, else takes the pages
        try:
            sig = self._signature(entries) if self.use_graphs and total <= self.graph_max_tokens else None
            fill, fill_first = self._decode_fill(entries) if sig is not None else (0, False)
            if fill:
                sig = ((1, (0,)),) * fill + sig if fill_first else sig + ((1, (0,)),) * fill
            if sig is not None:                           # a captured step is keyed by its shape and its context bucket
                sig = (sig, self._context_bucket(max(p0 + n for p0, n in zip(first, counts))))
            if sig is not None and self._graph_wanted(entries, total + fill, sig):
                logits = self._graph_step(entries, arrays, first, total + fill, sig, fill, fill_first)
                self.cache.retire(slots)
                self.steps += 1
                self._raise_if_not_finite()
                if fill and logits is not None:           # the scratch rows' logits are dropped
                    return logits[fill:] if fill_first else logits[:len(entries)]
                return logits
            rows_of, segments = self._rows(entries, arrays, first)
            if all(type(w) is list for w in wanted):       # (few places each: one short list)
                rows = np.array([seg[1] + w for seg, places in zip(segments, wanted) for w in places], dtype=np.int32)
            else:
                rows = np.concatenate([seg[1] + np.asarray(w, dtype=np.int64) for seg, w in zip(segments, wanted)]
                                      ).astype(np.int32)
            r = rows.size
            stateful = self.cache.has_state()
            parts = [rows_of.ravel(), rows]
            if stateful:
                parts.append(np.fromiter((seg[0] for seg in segments), np.int32, len(segments)))
            self._upload.send(np.concatenate(parts), self._meta)
            ctx = self.ctx
            ctx.begin_step()
            ctx.n_tokens = total
            ctx.token_ids = self._meta[0:total]
            ctx.positions = self._meta[total:2 * total]
            ctx.slots = self._meta[2 * total:3 * total]
            ctx.segments = segments
            ctx.single_tokens = total == len(entries)
            ctx.max_context = max(p0 + n for (_, _, n, p0) in segments)
            want_rows = self._meta[3 * total:3 * total + r] if r else None
            ctx.segment_slots = self._meta[3 * total + r:3 * total + r + len(segments)] if stateful else None
            logits = self.model.forward(ctx, want_rows)
            self.cache.retire(slots)
            self.steps += 1
            self._raise_if_not_finite()
            return logits
        except Exception:
            self.poisoned = True
            raise

    def _raise_if_not_finite(self):
        if not self.check_finite:
            return
        bits, where = self._status.tolist()               # (waits for the step: the price of the mode)
        if bits:
            kinds = " and ".join(name for bit, name in ((1, "a NaN"), (2, "an infinity")) if bits & bit)
            raise NonFiniteHidden(f"the hidden state holds {kinds}: first after layer run {where >> 20}, "
                                  f"batch row {where & 0xFFFFF}")

    # -- reports -------------------------------------------------------------------------------
    def memory_report(self):
        """The plan beside what is held now, in bytes."""
        actual = dict(weights=self.model.arena.used if self.model.arena is not None else self.model.weight_bytes(),
                      kv_pages=self.cache.kv_bytes(), block_tables=self.cache.table_bytes(),
                      state=self.cache.state_bytes(), workspace=self.workspace.planned_bytes,
                      workspace_beyond_plan=self.workspace.unplanned_bytes(),
                      metadata=self._meta.numel() * 4 + self._status.numel() * 4,
                      library_scratch=self.kernels.library_workspace_bytes())
        return {"planned": self.memory_plan.as_dict(), "actual": actual}

    def profile_report(self, reset=False):
        """Time per kernel class since the runner was built (or the last reset); None without profile=True."""
        profiler = self.kernels.profiler
        if profiler is None:
            return None
        report = profiler.report()
        if reset:
            profiler.reset()
        return report
