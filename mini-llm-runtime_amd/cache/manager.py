"""The cache manager: pages of keys and values with a block table per request, and slots of
fixed-size state per request.

A model names its cache needs as one spec per cache entry (an entry is what one run of a layer
reads and writes): `PagedSpec` for a mixer that keeps something per token (`KvSpec`, keys and
values, is the usual case of it), `StateSpec` for a mixer with state of fixed size, None for a
layer without memory.  What a page holds is the mixer's business: the spec names the tensors
and their shape within a page, the manager only multiplies them out.  Entries with equal specs
form a group; a group has its own pool of pages (one page id is valid in every entry of the
group), its own page size, its own block tables and its own rule for giving pages back (all
tokens kept, or only a window).  The bookkeeping itself (free lists, tables, lengths, invariants) is native code in
csrc/host/cache_manager.cpp; this module owns the device memory and keeps the device copies
of the block tables current.

Device layout of a group: keys [entries, num_pages, kv_heads, page_size, head_dim]; values transposed
within a page, [entries, num_pages, kv_heads, head_dim, page_size], so that the keys of one channel lie
side by side for the matrix-core product of probabilities and values;
block table int32 [max_slots, max_blocks], -1 where no page is mapped.  Unused memory is
filled with NaN so that a read of a never-written key shows (the reference fills its cache
with 0xFF for the same reason, src/minillm/cuda/storage.cpp:199-200).
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Optional, Tuple

import numpy as np
import torch

from ..kernels import build


class CacheError(RuntimeError):
    pass


class CacheFull(CacheError):
    """Not enough free pages (or slots) for what was asked; nothing was changed."""


PAGE = "page"          # stands for the page's tokens in a `PagedSpec` shape


@dataclass(frozen=True)
class PagedSpec:
    """What a mixer keeps per token: named tensors, each given by its shape WITHIN a page, with `PAGE` where
    the page's tokens go; the manager allocates [pages + 1, *shape] of each for every entry of the group.
    `page_size` None: the engine's; `dtype` None: the engine's element type."""
    tensors: Tuple[Tuple[str, Tuple], ...]
    window: Optional[int] = None      # None: all tokens are kept
    page_size: Optional[int] = None
    dtype: Optional[torch.dtype] = None

    def shape_of(self, name, page_size):
        for n, shape in self.tensors:
            if n == name:
                return tuple(page_size if e == PAGE else int(e) for e in shape)
        raise KeyError(name)

    def elements_per_page(self, page_size):
        total = 0
        for name, _ in self.tensors:
            count = 1
            for e in self.shape_of(name, page_size):
                count *= e
            total += count
        return total


@dataclass(frozen=True)
class KvSpec:
    """Keys [kv_heads, page, head_dim] and values [kv_heads, head_dim, page]: transposed within the page,
    so that the keys of one channel lie side by side for the matrix-core product of probabilities and
    values."""
    kv_heads: int
    head_dim: int
    window: Optional[int] = None      # None: all keys are kept

    def paged(self):
        return PagedSpec((("k", (self.kv_heads, PAGE, self.head_dim)), ("v", (self.kv_heads, self.head_dim, PAGE))),
                         self.window)


def _as_paged(spec):
    if isinstance(spec, KvSpec):
        return spec.paged()
    return spec if isinstance(spec, PagedSpec) else None


@dataclass(frozen=True)
class StateSpec:
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class PagedView:
    tensors: dict                     # name -> [num_pages + 1, *shape within a page] (the last page: scratch)
    block_table: torch.Tensor         # device int32 [max_slots + 1, max_blocks] (the last row: the scratch request)
    page_size: int
    window: Optional[int]
    group: int


@dataclass
class KvView:
    k_pages: torch.Tensor             # [num_pages + 1, kv_heads, page_size, head_dim] (the last page: scratch)
    v_pages: torch.Tensor             # [num_pages + 1, kv_heads, head_dim, page_size]
    block_table: torch.Tensor         # device int32 [max_slots + 1, max_blocks] (the last row: the scratch request)
    page_size: int
    window: Optional[int]
    group: int


def _host_lib():
    lib = build.load("host")
    if not getattr(lib, "_mlr_typed", False):
        lib.mlr_cache_create.restype = ctypes.c_void_p
        lib.mlr_cache_create.argtypes = [ctypes.c_int, ctypes.c_int]
        lib.mlr_cache_destroy.argtypes = [ctypes.c_void_p]
        lib.mlr_cache_destroy.restype = None
        lib.mlr_cache_add_group.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        lib.mlr_cache_max_blocks.argtypes = [ctypes.c_void_p, ctypes.c_int]
        lib.mlr_cache_free_pages.argtypes = [ctypes.c_void_p, ctypes.c_int]
        lib.mlr_cache_free_slots.argtypes = [ctypes.c_void_p]
        lib.mlr_cache_table.argtypes = [ctypes.c_void_p, ctypes.c_int]
        lib.mlr_cache_table.restype = ctypes.POINTER(ctypes.c_int32)
        lib.mlr_cache_length.argtypes = [ctypes.c_void_p, ctypes.c_int]
        lib.mlr_cache_acquire_slot.argtypes = [ctypes.c_void_p]
        lib.mlr_cache_release_slot.argtypes = [ctypes.c_void_p, ctypes.c_int]
        i32p = ctypes.POINTER(ctypes.c_int32)
        intp = ctypes.POINTER(ctypes.c_int)
        lib.mlr_cache_prepare.argtypes = [ctypes.c_void_p, i32p, i32p, ctypes.c_int, intp, intp]
        lib.mlr_cache_commit.argtypes = [ctypes.c_void_p, i32p, i32p, ctypes.c_int]
        lib.mlr_cache_commit_first.argtypes = [ctypes.c_void_p, i32p, i32p, ctypes.c_int, i32p]
        lib.mlr_cache_retire.argtypes = [ctypes.c_void_p, i32p, ctypes.c_int]
        lib.mlr_cache_take_dirty.argtypes = [ctypes.c_void_p, ctypes.c_int, i32p]
        lib.mlr_cache_check.argtypes = [ctypes.c_void_p]
        lib._mlr_typed = True
    return lib


def _i32(values):
    arr = np.ascontiguousarray(values, dtype=np.int32)
    return arr, arr.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))


class PageBook:
    """The native bookkeeping alone (no device memory): usable and testable without a GPU."""

    def __init__(self, max_slots, max_length):
        self._lib = _host_lib()
        self._h = self._lib.mlr_cache_create(max_slots, max_length)
        if not self._h:
            raise CacheError("max_slots and max_length must be positive")
        self.max_slots, self.max_length = max_slots, max_length
        self.groups = []                  # (page_size, num_pages, window)

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.mlr_cache_destroy(h)

    def add_group(self, page_size, num_pages, window=None):
        g = self._lib.mlr_cache_add_group(self._h, page_size, num_pages, window or 0)
        if g < 0:
            raise CacheError("page_size and num_pages must be positive")
        self.groups.append((page_size, num_pages, window))
        return g

    def max_blocks(self, group):
        return self._lib.mlr_cache_max_blocks(self._h, group)

    def free_pages(self, group=0):
        return self._lib.mlr_cache_free_pages(self._h, group)

    def free_slots(self):
        return self._lib.mlr_cache_free_slots(self._h)

    def table(self, group=0):
        """Host view [max_slots, max_blocks] of the group's block table (not a copy)."""
        ptr = self._lib.mlr_cache_table(self._h, group)
        return np.ctypeslib.as_array(ptr, shape=(self.max_slots, self.max_blocks(group)))

    def length(self, slot):
        n = self._lib.mlr_cache_length(self._h, slot)
        if n < 0:
            raise CacheError(f"slot {slot} is not live")
        return n

    def acquire_slot(self):
        s = self._lib.mlr_cache_acquire_slot(self._h)
        if s < 0:
            raise CacheFull("no free request slot")
        return s

    def release_slot(self, slot):
        if self._lib.mlr_cache_release_slot(self._h, slot) != 0:
            raise CacheError(f"slot {slot} is not live (released twice?)")

    def _raise(self, rc, group, need_free):
        if rc == -1:
            raise CacheError("batch names a slot that is not live")
        if rc == -2:
            raise CacheError(f"a request would grow beyond max_length {self.max_length}")
        if rc == -3:
            raise CacheFull(f"cache group {group} needs {need_free[0]} more pages but only "
                            f"{need_free[1]} are free")
        if rc == -4:
            raise CacheError("a batch entry must bring at least one token")
        if rc == -5:
            raise CacheError("a slot appears twice in one batch")
        raise CacheError(f"cache bookkeeping failed ({rc})")

    def prepare(self, slots, counts):
        """Raises if the batch {slot: number of new tokens} cannot be taken; changes nothing."""
        s, sp = _i32(slots)
        c, cp = _i32(counts)
        group = ctypes.c_int(-1)
        need_free = (ctypes.c_int * 2)(0, 0)
        rc = self._lib.mlr_cache_prepare(self._h, sp, cp, len(s), ctypes.byref(group), need_free)
        if rc != 0:
            self._raise(rc, group.value, need_free)

    def commit(self, slots, counts):
        self.prepare(slots, counts)
        s, sp = _i32(slots)
        c, cp = _i32(counts)
        rc = self._lib.mlr_cache_commit(self._h, sp, cp, len(s))
        if rc != 0:
            self._raise(rc, -1, (0, 0))

    def commit_first(self, slots, counts):
        """`commit`, returning each entry's first position (the slot's length before the batch).  Raises
        like `prepare`, with nothing changed."""
        s, sp = _i32(slots)
        c, cp = _i32(counts)
        first = np.empty(len(s), dtype=np.int32)
        rc = self._lib.mlr_cache_commit_first(self._h, sp, cp, len(s), first.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)))
        if rc != 0:
            self.prepare(slots, counts)           # raises the precise error
            self._raise(rc, -1, (0, 0))
        return first.tolist()

    def retire(self, slots):
        s, sp = _i32(slots)
        rc = self._lib.mlr_cache_retire(self._h, sp, len(s))
        if rc < 0:
            raise CacheError("retire names a slot that is not live")
        return rc

    def take_dirty(self, group=0):
        out = np.empty(self.max_slots, dtype=np.int32)
        n = self._lib.mlr_cache_take_dirty(self._h, group, out.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)))
        return out[:n].tolist()

    def check(self):
        rc = self._lib.mlr_cache_check(self._h)
        if rc != 0:
            raise CacheError(f"page bookkeeping invariant {rc} is broken")


class CacheManager:
    """Device memory for every cache entry of a model plus the bookkeeping above."""

    @staticmethod
    def plan(entry_specs, dtype, page_size, max_tokens, max_slots, max_length):
        """(bytes of pages, of block tables, of state slabs) that a manager with these sizes allocates:
        per group of equal specs every tensor of the spec as [entries, pages + 1, *shape within a page]
        and a table [max_slots + 1, ceil(max_length / page size)] of int32; per `StateSpec` two slabs
        [max_slots + 1, *shape] (live and staged)."""
        groups = {}
        state = 0
        for spec in entry_specs:
            paged = _as_paged(spec)
            if paged is not None:
                groups[paged] = groups.get(paged, 0) + 1
            elif isinstance(spec, StateSpec):
                count = 2 * (max_slots + 1)          # live and staged rows, one more for the scratch request
                for extent in spec.shape:
                    count *= int(extent)
                state += count * torch.empty((), dtype=spec.dtype).element_size()
        kv = tables = 0
        for spec, n in groups.items():
            size = spec.page_size or page_size
            element = torch.empty((), dtype=spec.dtype or dtype).element_size()
            pages = (max_tokens + size - 1) // size + 1
            kv += n * pages * spec.elements_per_page(size) * element
            tables += (max_slots + 1) * ((max_length + size - 1) // size) * 4
        return kv, tables, state

    @staticmethod
    def tokens_that_fit(entry_specs, dtype, page_size, max_slots, max_length, budget_bytes):
        """The largest pool (in tokens: a multiple of every group's page size) whose pages, tables and state fit
        `budget_bytes`, at most what `max_slots` requests of `max_length` tokens can hold; 0 when not even one
        unit fits.  What the reference calls kv_capacity_tokens (include/minillm/cuda/runtime.h:28), here derived
        from the budget instead of asked of the user."""
        import math
        unit = 1
        for spec in entry_specs:
            paged = _as_paged(spec)
            if paged is not None:
                size = paged.page_size or page_size
                unit = unit * size // math.gcd(unit, size)
        most = max_slots * (-(-max_length // unit))          # units that the slots can hold at all
        fits = lambda units: sum(CacheManager.plan(entry_specs, dtype, page_size, units * unit, max_slots, max_length)) <= budget_bytes
        if fits(most):
            return most * unit
        lo, hi = 0, most                                     # fits(lo) (or lo == 0), not fits(hi)
        while hi - lo > 1:
            mid = (lo + hi) // 2
            lo, hi = (mid, hi) if fits(mid) else (lo, mid)
        return lo * unit if lo > 0 and fits(lo) else 0

    def __init__(self, entry_specs, dtype, device, page_size, max_tokens, max_slots, max_length):
        if page_size <= 0 or max_tokens <= 0:
            raise CacheError("page_size and max_tokens must be positive")
        self.dtype, self.device, self.page_size = dtype, torch.device(device), page_size
        self.max_slots, self.max_length = max_slots, max_length
        self.book = PageBook(max_slots, max_length)
        self.entry_specs = list(entry_specs)
        self._group_of_spec = {}
        self._entry_place = {}            # cache id -> (group, index within the group)
        members = []
        self.group_specs, self.group_page_size, self.group_pages = [], [], []
        for cid, spec in enumerate(self.entry_specs):
            paged = _as_paged(spec)
            if paged is None:
                continue
            if paged not in self._group_of_spec:
                size = paged.page_size or page_size
                if size <= 0:
                    raise CacheError("a group's page size must be positive")
                pages = (max_tokens + size - 1) // size
                self._group_of_spec[paged] = self.book.add_group(size, pages, paged.window)
                members.append([])
                self.group_specs.append(paged)
                self.group_page_size.append(size)
                self.group_pages.append(pages)
            g = self._group_of_spec[paged]
            self._entry_place[cid] = (g, len(members[g]))
            members[g].append(cid)
        self.num_pages = self.group_pages[0] if self.group_pages else (max_tokens + page_size - 1) // page_size
        # Beyond the pool and the slots of the bookkeeping, every group has one page more, every block
        # table one row more and every state slab one row more: a scratch request of one token (slot
        # `scratch_slot`, its only block mapped to that page), with which a step may fill a batch up to a
        # size it has a captured graph for.
        self.scratch_slot = max_slots
        self._paged, self._tables = [], []      # per group: {name: [entries, pages + 1, *shape]}, block table
        for g, spec in enumerate(self.group_specs):
            size, pages = self.group_page_size[g], self.group_pages[g]
            kind = spec.dtype or dtype
            fill = float("nan") if kind.is_floating_point else 0
            self._paged.append({name: torch.full((len(members[g]), pages + 1, *spec.shape_of(name, size)), fill,
                                                 dtype=kind, device=self.device)
                                for name, _ in spec.tensors})
            table = torch.full((max_slots + 1, self.book.max_blocks(g)), -1, dtype=torch.int32, device=self.device)
            table[max_slots, 0] = pages
            self._tables.append(table)
        self._stages = {}                # group -> [pinned copy of its table, event of the last upload, in use]
        # State of fixed size: a live slab, which mixers read, and a staged one, into which they write the
        # state their step leads to; the staged rows of a step's requests become live when every layer has
        # run (`commit_state`), so a step that fails on the way leaves the live state as it was.
        self._states, self._staged = {}, {}
        for cid, spec in enumerate(self.entry_specs):
            if isinstance(spec, StateSpec):
                self._states[cid] = torch.zeros((max_slots + 1, *spec.shape), dtype=spec.dtype, device=self.device)
                self._staged[cid] = torch.zeros_like(self._states[cid])

    # -- views for the parts ---------------------------------------------------------------------
    def paged_view(self, cache_id):
        """What the entry keeps per token: its tensors [pages + 1, *shape within a page], the group's block
        table, page size and window."""
        g, i = self._entry_place[cache_id]
        spec = self.group_specs[g]
        return PagedView({name: t[i] for name, t in self._paged[g].items()}, self._tables[g],
                         self.group_page_size[g], spec.window, g)

    def kv_view(self, cache_id):
        """The same for an entry of keys and values (`KvSpec`)."""
        g, i = self._entry_place[cache_id]
        spec = self.group_specs[g]
        return KvView(self._paged[g]["k"][i], self._paged[g]["v"][i], self._tables[g], self.group_page_size[g],
                      spec.window, g)

    def state_view(self, cache_id):
        """[max_slots + 1, *shape]: the requests' live state (row = slot); read it, do not write it."""
        return self._states[cache_id]

    def state_stage(self, cache_id):
        """[max_slots + 1, *shape]: where a mixer leaves the state that its step leads to, in the rows of the
        step's slots (every slot of the step, in every step that writes the entry)."""
        return self._staged[cache_id]

    def has_state(self):
        return bool(self._states)

    def commit_state(self, segment_slots):
        """The staged rows of the step's requests (`segment_slots`: device integer vector, one slot per
        entry of the batch) become live.  Device work only, so a captured step holds it.  The scratch
        request's state starts every step at zero."""
        index = segment_slots.long()
        for cid, live in self._states.items():
            live.index_copy_(0, index, self._staged[cid].index_select(0, index))
            live[self.max_slots].zero_()

    def snapshot_state(self):
        return {cid: live.clone() for cid, live in self._states.items()}

    def restore_state(self, snapshot):
        for cid, saved in snapshot.items():
            self._states[cid].copy_(saved)

    def reserve_unit(self):
        """Tokens in which a request's whole life can be set aside so that every group has the pages for it:
        the least common multiple of the groups' page sizes (with one group, its page size)."""
        import math
        unit = 1
        for size in self.group_page_size or [self.page_size]:
            unit = unit * size // math.gcd(unit, size)
        return unit

    def paged_tensors(self):
        """Every group's tensors, [entries, pages + 1, *shape within a page] each (a benchmark fills them with
        noise instead of running a prompt)."""
        return [t for group in self._paged for t in group.values()]

    def kv_bytes(self):
        return sum(t.numel() * t.element_size() for t in self.paged_tensors())

    def table_bytes(self):
        return sum(t.numel() * t.element_size() for t in self._tables)

    def state_bytes(self):
        return sum(t.numel() * t.element_size() for t in list(self._states.values()) + list(self._staged.values()))

    # -- requests --------------------------------------------------------------------------------
    def acquire_slot(self):
        slot = self.book.acquire_slot()
        for state in self._states.values():
            state[slot].zero_()
        return slot

    def release_slot(self, slot):
        self.book.release_slot(slot)

    def length(self, slot):
        return self.book.length(slot)

    def free_pages(self, group=0):
        return self.book.free_pages(group)

    def prepare(self, slots, counts):
        self.book.prepare(slots, counts)

    def commit(self, slots, counts):
        self.book.commit(slots, counts)
        self.sync_tables()

    def commit_first(self, slots, counts):
        first = self.book.commit_first(slots, counts)
        self.sync_tables()
        return first

    def retire(self, slots):
        """After a step: give back what windows have passed.  The device tables are brought up
        to date before the next step (commit)."""
        return self.book.retire(slots)

    def sync_tables(self):
        """Changed rows of the block tables go to the device through a pinned staging copy of the table, with
        asynchronous copies on the current stream (a copy from pageable memory would block the host on every
        step that crosses a page's edge); an event guards the staging rows until the copies have left them."""
        for g, dev in enumerate(self._tables):
            rows = self.book.take_dirty(g)
            if not rows:
                continue
            host = torch.from_numpy(self.book.table(g))
            if dev.device.type != "cuda":
                dev[:self.max_slots].copy_(host)
                continue
            stage = self._stages.get(g)
            if stage is None:
                stage = self._stages[g] = [torch.empty(tuple(host.shape), dtype=torch.int32).pin_memory(),
                                           torch.cuda.Event(), False]
            pinned, event, busy = stage
            if busy:
                event.synchronize()
            if len(rows) * 4 >= self.max_slots:
                pinned.copy_(host)
                dev[:self.max_slots].copy_(pinned, non_blocking=True)
            else:
                for s in rows:
                    pinned[s].copy_(host[s])
                    dev[s].copy_(pinned[s], non_blocking=True)
            event.record()
            stage[2] = True

    def check(self):
        self.book.check()
