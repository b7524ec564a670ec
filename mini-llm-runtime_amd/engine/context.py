"""What a part may see of the running step, and the scratch memory it may use."""
from __future__ import annotations

import numpy as np
import torch


class Workspace:
    """Named scratch buffers that live as long as the runner.  `reserve` carves every buffer that the
    parts have named for the largest step out of ONE allocation; a name that was not planned (a part
    without a plan), or a size beyond its plan, is allocated when it is first asked for and grows only
    when a larger size is asked, so steady steps allocate nothing either way."""

    def __init__(self, device):
        self.device = torch.device(device)
        self._buffers = {}
        self._arena = None
        self.planned_bytes = 0
        self._unplanned = {}          # (name, dtype) -> bytes allocated outside the plan
        self._views = {}              # (name, dtype, shape) -> the view handed out for it

    @staticmethod
    def plan_bytes(plan):
        """plan: {(name, dtype): elements}.  Bytes of the one allocation that holds them (256-byte places)."""
        return sum(-(-count * torch.empty((), dtype=dtype).element_size() // 256) * 256
                   for (_, dtype), count in plan.items())

    def reserve(self, plan):
        total = self.plan_bytes(plan)
        self._arena = torch.empty(max(total, 1), dtype=torch.uint8, device=self.device)
        self.planned_bytes = total
        at = 0
        for (name, dtype), count in plan.items():
            size = count * torch.empty((), dtype=dtype).element_size()
            self._buffers[(name, dtype)] = self._arena[at:at + size].view(dtype)
            at += -(-size // 256) * 256

    def unplanned_bytes(self):
        return sum(self._unplanned.values())

    def get(self, name, shape, dtype):
        # (a step asks for the same few shapes again and again: the views are kept, a steady step makes none)
        shape = tuple(shape)
        view = self._views.get((name, dtype, shape))
        if view is not None:
            return view
        count = 1
        for extent in shape:
            count *= int(extent)
        key = (name, dtype)
        buf = self._buffers.get(key)
        if buf is None or buf.numel() < count:
            buf = torch.empty(max(count, 1), dtype=dtype, device=self.device)
            self._buffers[key] = buf
            self._unplanned[key] = buf.numel() * buf.element_size()
            for stale in [k for k in self._views if k[0] == name and k[1] == dtype]:
                del self._views[stale]                     # (views of the buffer that this one replaces)
        view = buf[:count].view(shape)
        if len(self._views) >= 4096:
            self._views.clear()
        self._views[(name, dtype, shape)] = view
        return view

    def bytes(self):
        return self.planned_bytes + self.unplanned_bytes()

    def buffers(self):
        """The buffers as they are now.  A captured graph holds on to this list: it keeps using the
        memory it was captured with, also after a larger step has made a name's buffer grow."""
        return list(self._buffers.values())


class Uploader:
    """Small host-to-device copies through one pinned buffer.  The copy is asynchronous; an event
    guards the buffer so that the next use waits until the previous copy has left it."""

    def __init__(self, capacity, device):
        self.device = torch.device(device)
        self._host = torch.empty(capacity, dtype=torch.int32).pin_memory()
        self._event = torch.cuda.Event()
        self._busy = False

    def send(self, values, dst):
        """values: a list of ints or an int32 numpy vector; dst: device int32 vector of at least that many elements."""
        n = len(values)
        if n > self._host.numel():
            if self._busy:
                self._event.synchronize()
                self._busy = False
            self._host = torch.empty(max(n, 2 * self._host.numel()), dtype=torch.int32).pin_memory()
        if self._busy:
            self._event.synchronize()
        if isinstance(values, np.ndarray):
            self._host.numpy()[:n] = values               # (a view of the pinned buffer: one copy, no tensor made)
        else:
            self._host[:n] = torch.tensor(values, dtype=torch.int32)
        dst[:n].copy_(self._host[:n], non_blocking=True)
        self._event.record()
        self._busy = True


class StepContext:
    """One step's view for the parts: the tokens with their positions and slots (device int32
    vectors of equal length), the segments they form (host), the cache, the kernels and the
    scratch memory."""

    def __init__(self, kernels, cache, workspace, dtype, max_positions, split_keys, split_max_tokens):
        self.kernels, self.cache, self.workspace, self.dtype = kernels, cache, workspace, dtype
        self.max_positions = max_positions
        self.split_keys, self.split_max_tokens = split_keys, split_max_tokens
        self.target_workgroups = 512      # about two workgroups per compute unit
        self.compute_units = (torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count
                              if torch.cuda.is_available() else 1)
        self.n_tokens = 0
        self.token_ids = self.positions = self.slots = None
        self.segments = []            # (slot, first row, number of tokens, first position)
        self.segment_slots = None     # device int32, one slot per segment (set when the model keeps state per request)
        self.single_tokens = False    # every segment brings exactly one token (a decoding step)
        self.max_context = 0          # largest position + 1 among the step's tokens
        self._groups = {}
        self._group_upload = None
        self.fixed_groups = None      # a captured step's groups: {key: token_groups' result}, in tensors of their own
        self.status = None            # device int32 [2] when the hidden state is to be checked after every layer
        self.partial_budget = None    # floats that split attention's partial results may take (the memory plan's)

    def begin_step(self):
        self._groups = {}
        self.fixed_groups = None

    def token_groups(self, tokens_per_group, big_factor=0):
        """The step's rows cut into groups of consecutive tokens of one request, as device int32 vectors
        (first row of each group, tokens in each group) with their number.  Returns (small, big, (rows in
        small groups, one beyond the last batch row of a small group)): small groups hold at most
        `tokens_per_group` tokens; with big_factor > 0, a request that brings more than `tokens_per_group`
        tokens is cut into big groups of at most big_factor * tokens_per_group instead (prompt portions), else
        `big` is empty."""
        key = (tokens_per_group, big_factor)
        hit = self._groups.get(key)
        if hit is not None:
            return hit
        if self.fixed_groups is not None and key in self.fixed_groups:
            return self.fixed_groups[key]
        first, count, big_first, big_count = [], [], [], []
        small_rows = small_end = 0
        for _, row, n, _ in self.segments:
            if big_factor > 0 and n > tokens_per_group:
                size = big_factor * tokens_per_group
                for i in range(0, n, size):
                    big_first.append(row + i)
                    big_count.append(min(size, n - i))
            else:
                small_rows += n
                small_end = max(small_end, row + n)
                for i in range(0, n, tokens_per_group):
                    first.append(row + i)
                    count.append(min(tokens_per_group, n - i))
        g, gb = len(first), len(big_first)
        if self.fixed_groups is not None:
            # a step that is to be captured: its groups depend on the lengths of its entries only, so they
            # get a tensor of their own once (this is the eager run before the capture) and stay there
            dev = torch.tensor(first + count + big_first + big_count + [0], dtype=torch.int32, device=self.workspace.device)
        else:
            dev = self.workspace.get(f"token_groups_{tokens_per_group}_{big_factor}", (2 * (g + gb),), torch.int32)
            if self._group_upload is None:
                self._group_upload = Uploader(4096, dev.device)
            self._group_upload.send(first + count + big_first + big_count, dev)
        hit = ((dev[:g], dev[g:2 * g], g), (dev[2 * g:2 * g + gb], dev[2 * g + gb:2 * g + 2 * gb], gb),
               (small_rows, small_end))
        if self.fixed_groups is not None:
            self.fixed_groups[key] = hit
        self._groups[key] = hit
        return hit

    def attention_split(self, rows, batch_rows, kv_heads, q_heads, head_dim, longest=None):
        """(split_keys, max_splits, partial buffer).  A batch of many tokens fills the GPU with one
        workgroup per (token group, kv head); a small batch over long contexts does not, so there the
        keys of a token are split over several workgroups, in ranges [s * split_keys, (s + 1) *
        split_keys) of absolute key positions, and merged in ascending order.  split_keys is the
        largest of base, 2 base, 4 base, ... that still gives `target_workgroups`; what a token's
        result is does not depend on the choice beyond rounding.  `rows` tokens take part; the partial
        results are indexed by batch row, of which there are `batch_rows`.  `longest`: the most keys a
        workgroup of the kernel can walk without a split; a longer context is split whatever the batch."""
        forced = longest is not None and self.max_context > longest
        if rows > self.split_max_tokens and not forced:
            return 0, 1, None
        return self._split(max(1, rows * kv_heads), self.target_workgroups, batch_rows, q_heads, head_dim, longest)

    def group_split(self, groups, batch_rows, kv_heads, q_heads, head_dim, longest=None):
        """As `attention_split` for `groups` groups of many tokens each (prompt portions), which give
        one workgroup per (group, kv head).  `longest`: the most keys a workgroup can take without a
        split; a longer context is split whatever the number of groups."""
        return self._split(max(1, groups * kv_heads), self.compute_units, batch_rows, q_heads, head_dim, longest)

    def fixed_split(self, rows, q_heads, head_dim):
        """(split_keys, max_splits, rows a launch, partial buffer) for the attention kernel whose results must
        not depend on the batch by a single bit (the float engine's): a token's keys are always cut into ranges
        of `split_keys` of the runner's setting, whatever else the step holds, so the sums that make up its
        result and their order follow from its own position alone.  (A context of more than 1024 ranges
        doubles their width: the merge kernel's limit.)  The partial results of all rows may exceed what was
        planned for them; then the rows are served by several launches."""
        base = self.split_keys
        if base <= 0 or self.max_context <= base:
            return 0, 1, rows, None
        keys = base
        while -(-self.max_context // keys) > 1024:
            keys *= 2
        max_splits = -(-self.max_context // keys)
        per_row = self.kernels.attention_partial_numel(1, q_heads, head_dim, max_splits)
        chunk = rows if self.partial_budget is None else max(1, min(rows, self.partial_budget // per_row))
        return keys, max_splits, chunk, self.workspace.get("attn_partial", (chunk * per_row,), torch.float32)

    @staticmethod
    def forced_splits(max_length, base, longest):
        """Key splits that a context of `max_length` needs at least when one workgroup walks at most `longest`
        keys: ranges of the largest of base, 2 base, 4 base, ... that `longest` holds (1: no split needed)."""
        if longest is None or max_length <= longest or base <= 0:
            return 1
        keys = base
        while keys * 2 <= longest:
            keys *= 2
        return -(-max_length // keys)

    def _split(self, units, enough, batch_rows, q_heads, head_dim, longest=None):
        """`units` workgroups without a split; no split when they are `enough`.  The partial results never take
        more than `partial_budget` floats (when one is set: the runner's memory plan): key ranges are doubled
        until they fit, which a forced split allows up to `longest`."""
        base = self.split_keys
        forced = longest is not None and self.max_context > longest
        if base <= 0 or (self.max_context <= base and not forced):
            return 0, 1, None
        keys = base
        while keys * 2 < self.max_context and units * (-(-self.max_context // (keys * 2))) >= self.target_workgroups:
            keys *= 2
        if forced:
            while keys > base and keys > longest:
                keys //= 2
        elif units >= enough:
            return 0, 1, None
        budget = self.partial_budget
        numel = lambda k: self.kernels.attention_partial_numel(batch_rows, q_heads, head_dim, -(-self.max_context // k))
        while budget is not None and numel(keys) > budget and (not forced or keys * 2 <= longest):
            if keys >= self.max_context:                 # one range holds every key: no split, nothing to keep
                return 0, 1, None
            keys *= 2
        max_splits = -(-self.max_context // keys)
        if max_splits <= 1:
            return 0, 1, None
        while max_splits > 1024:                     # the merge kernels' limit
            keys *= 2
            max_splits = -(-self.max_context // keys)
        numel = self.kernels.attention_partial_numel(batch_rows, q_heads, head_dim, max_splits)
        return keys, max_splits, self.workspace.get("attn_partial", (numel,), torch.float32)
