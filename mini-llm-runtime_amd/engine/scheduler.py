"""The scheduler above the step function: admission, portions of prompts under a token budget,
decoding, finishing and freeing.  It follows the reference's engine loop
(src/engine.cpp:295-355 admission, 392-580 iteration; src/scheduler.cpp:11-49 batch forming):

  * submit refuses what can never run: an empty prompt, ids outside the vocabulary,
    max_tokens < 1, prompt + max_tokens beyond max_model_len or beyond the whole pool;
  * admission is first-come within aged priority; a request is admitted when a slot is free
    and pages for its WHOLE life, ceil((prompt + max_tokens) / page_size), can be set aside.
    Because everything is set aside up front, pages cannot run out in the middle of a
    request: a request that does not fit waits until others finish and free theirs;
    after `admission_reserve_ms` of waiting the oldest request may no longer be overtaken;
  * each iteration gives every decoding request one token and fills the rest of the token
    budget with portions of prompts (policy mixed), or runs prompts first (prefill_first);
    the batch-forming decision itself is native (csrc/host/scheduler.cpp);
  * the last token of a prompt and every decoded token ask for logits; a request ends on an
    end-of-sequence id (unless ignore_eos) or at max_tokens, and its pages and slot are
    given back at once.
"""
from __future__ import annotations

import ctypes
import time
from dataclasses import dataclass, field
from typing import List, Optional

from ..kernels import build
from ..sampling import RequestRng, Sampler
from .step import Entry, Runner


class _Item(ctypes.Structure):
    _fields_ = [("key", ctypes.c_int64), ("prefill_remaining", ctypes.c_int64), ("priority", ctypes.c_int32),
                ("wait_ms", ctypes.c_int64), ("order", ctypes.c_uint64)]


class _Slice(ctypes.Structure):
    _fields_ = [("key", ctypes.c_int64), ("tokens", ctypes.c_int64), ("prefill", ctypes.c_int32)]


class _Waiting(ctypes.Structure):
    _fields_ = [("pages", ctypes.c_int64), ("priority", ctypes.c_int32), ("waited_ms", ctypes.c_int64),
                ("order", ctypes.c_uint64)]


POLICIES = {"mixed": 0, "prefill_first": 1}


def _lib():
    lib = build.load("host")
    if not getattr(lib, "_mlr_sched_typed", False):
        lib.mlr_schedule_batch.argtypes = [ctypes.POINTER(_Item), ctypes.c_int, ctypes.c_int64, ctypes.c_int64,
                                           ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.POINTER(_Slice)]
        lib.mlr_effective_priority.argtypes = [ctypes.c_int, ctypes.c_int64, ctypes.c_int]
        lib.mlr_effective_priority.restype = ctypes.c_int64
        lib.mlr_admit.argtypes = [ctypes.POINTER(_Waiting), ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                  ctypes.c_int64, ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int32),
                                  ctypes.POINTER(ctypes.c_int64)]
        lib._mlr_sched_typed = True
    return lib


def effective_priority(priority, wait_ms, aging_ms):
    return _lib().mlr_effective_priority(priority, int(wait_ms), aging_ms)


def admit(items, free_pages, free_slots, aging_ms=250, reserve_ms=2000):
    """items: (pages of the request's whole life, priority, waited_ms, order) of every waiting request.  Returns
    (the queue's indices in the order of the walk, the indices that start now in that order, how many did not
    fit): see `mlr_admit`."""
    n = len(items)
    arr = (_Waiting * max(n, 1))()
    for i, (pages, priority, waited_ms, order) in enumerate(items):
        arr[i] = _Waiting(pages, priority, int(waited_ms), order)
    walk, started = (ctypes.c_int32 * max(n, 1))(), (ctypes.c_int32 * max(n, 1))()
    waits = ctypes.c_int64(0)
    count = _lib().mlr_admit(arr, n, free_pages, free_slots, aging_ms, reserve_ms, walk, started, ctypes.byref(waits))
    if count < 0:
        raise ValueError("aging_ms must be positive, reserve_ms and free_pages not negative")
    return list(walk[:n]), list(started[:count]), waits.value


def schedule_batch(items, batch_tokens, prefill_chunk, policy="mixed", aging_ms=250, portion_step=0):
    """items: (key, prefill_remaining, priority, wait_ms, order) each.  Returns the slices
    [(key, tokens, is_prefill)] of the next batch.  portion_step > 1: portions that do not end their
    prompt are multiples of it (the reference has no such thing: 0 gives its decision)."""
    if policy not in POLICIES:
        raise ValueError(f"policy must be one of {sorted(POLICIES)}")
    n = len(items)
    arr = (_Item * max(n, 1))()
    for i, (key, remaining, priority, wait_ms, order) in enumerate(items):
        arr[i] = _Item(key, remaining, priority, int(wait_ms), order)
    out = (_Slice * max(n, 1))()
    count = _lib().mlr_schedule_batch(arr, n, batch_tokens, prefill_chunk, POLICIES[policy], aging_ms,
                                      portion_step, out)
    if count < 0:
        raise ValueError("batch_tokens, prefill_chunk and aging_ms must be positive, portion_step not negative")
    return [(out[i].key, out[i].tokens, bool(out[i].prefill)) for i in range(count)]


@dataclass
class EngineOptions:
    """Names after the reference's EngineConfig (include/llmserve/config.h:15-33).  Its defaults are the limits
    of a laptop GPU (a pool of 8192 tokens, 8 slots, steps of 256 tokens, portions of 128); here what is left
    None is taken from the model and the device when an engine is built (`resolved`): a 2048-token prompt is one
    step, and the pool is what the device's budget leaves room for."""
    context_tokens: Optional[int] = None   # tokens the page pool holds; None: what the device's budget leaves room
                                           # for, at most max_active requests of max_model_len tokens
    max_model_len: Optional[int] = None    # longest prompt + output of one request; None: the model's positions
    max_active: int = 64                   # request slots
    batch_tokens: Optional[int] = None     # token budget of one step; None: prefill_chunk + max_active
    prefill_chunk: int = 2048              # longest portion of one prompt in a step
    block_size: int = 16                   # tokens in a page
    aging_ms: int = 250
    admission_reserve_ms: int = 2000
    policy: str = "mixed"
    queue_capacity: int = 65536
    portion_step: int = 32            # ours: portions that do not end their prompt are multiples of this, so
                                      # that step shapes come again and are replayed as graphs (0: the
                                      # reference's exact portions)
    kv_dtype: str = "auto"            # the cache's element type: "auto" or the engine's own
                                      # (include/minillm/cuda/runtime.h:18-30 has the cache's type and capacity
                                      # beside the budget; another type than the engine's is refused)
    device_budget_bytes: Optional[int] = 0   # the user's cap on what the runner may allocate; 0: none beside the rule
                                             # min(80 % of free memory, free - 512 MiB); None: no gate at all

    def resolved(self, max_positions):
        """A copy with every None filled in, as far as that needs no device: max_model_len from the model,
        batch_tokens from the portion and the slots.  context_tokens may stay None (the runner sizes the pool)."""
        from dataclasses import replace
        limit = min(self.max_model_len or max_positions, max_positions)
        if self.max_model_len is None and self.context_tokens is not None:
            limit = min(limit, self.context_tokens)       # (no request outgrows the pool)
        chunk = self.prefill_chunk
        batch = self.batch_tokens
        if batch is None:
            batch = chunk + self.max_active
            if self.context_tokens is not None:
                batch = max(min(batch, self.context_tokens), self.max_active)
                chunk = min(chunk, batch)
        return replace(self, max_model_len=limit, batch_tokens=batch, prefill_chunk=chunk)

    def validate(self):
        """src/config.cpp:8-36, on resolved options (context_tokens may still be None)."""
        if self.max_model_len is None or self.batch_tokens is None:
            raise ValueError("validate() wants resolved options")
        pool = self.context_tokens
        if self.block_size <= 0 or (pool is not None and (pool <= 0 or pool % self.block_size != 0)):
            raise ValueError("context_tokens must be a positive multiple of block_size")
        if self.max_model_len < 2 or (pool is not None and self.max_model_len > pool):
            raise ValueError("max_model_len must be in [2, context_tokens]")
        if self.max_active <= 0 or self.batch_tokens < self.max_active or (pool is not None and self.batch_tokens > pool):
            raise ValueError("require 1 <= max_active <= batch_tokens <= context_tokens")
        if self.prefill_chunk <= 0 or self.prefill_chunk > self.batch_tokens or self.queue_capacity <= 0:
            raise ValueError("invalid prefill or queue limit")
        if self.aging_ms <= 0 or self.admission_reserve_ms <= 0:
            raise ValueError("invalid aging interval")
        if self.policy not in POLICIES:
            raise ValueError(f"policy must be one of {sorted(POLICIES)}")
        if self.portion_step < 0:
            raise ValueError("portion_step must not be negative")
        if self.kv_dtype not in ("auto", "bfloat16", "float32"):
            raise ValueError("kv_dtype must be auto, bfloat16 or float32")
        if self.device_budget_bytes is not None and self.device_budget_bytes < 0:
            raise ValueError("device_budget_bytes must not be negative")


@dataclass
class Request:
    id: int
    prompt: List[int]
    max_tokens: int
    temperature: float = 0.0
    seed: int = 0
    ignore_eos: bool = False
    priority: int = 0
    # state
    order: int = 0
    created: float = 0.0
    last_scheduled: float = 0.0
    slot: Optional[int] = None
    pages: int = 0                    # pages set aside for its whole life
    processed: int = 0                # prompt tokens already run
    generated: List[int] = field(default_factory=list)
    rng: Optional[RequestRng] = None
    finish_reason: Optional[str] = None
    deadline: Optional[float] = None  # on the engine's clock; None: no time limit
    cancelled: bool = False


class Engine:
    """Continuous batching over one `Runner`.  Single-threaded: the caller drives `step()`."""

    def __init__(self, model, options: EngineOptions = None, clock=time.monotonic, runner=None, sampler=None,
                 device_budget_bytes="options", check_finite=False, profile=False):
        """`device_budget_bytes` (default: the options' own), `check_finite`, `profile`: handed to the `Runner`
        that is built here (see there): the budget gate before the cache is allocated, the check of the hidden
        state after every layer, time per kernel class."""
        self.options = (options or EngineOptions()).resolved(model.spec.max_positions)
        self.options.validate()
        o = self.options
        if device_budget_bytes == "options":
            device_budget_bytes = o.device_budget_bytes
        self.model = model
        # (a step of the scheduler asks for at most one row of logits per request)
        self.runner = runner or Runner(model, max_tokens=o.context_tokens, max_slots=o.max_active,
                                       max_length=o.max_model_len,
                                       max_batch_tokens=o.batch_tokens, page_size=o.block_size,
                                       max_logits_rows=o.max_active, device_budget_bytes=device_budget_bytes,
                                       check_finite=check_finite, profile=profile, kv_dtype=o.kv_dtype)
        if o.context_tokens is None:                      # the pool that the runner sized from the device's budget
            o.context_tokens = getattr(self.runner, "max_tokens", None) or o.max_active * o.max_model_len
            o.validate()
        self.sampler = sampler or Sampler(self.runner.kernels, self.runner.device, max_rows=o.max_active)
        self.clock = clock
        # pages are set aside in units that every group of the cache can serve (its page size, when all
        # groups have the same)
        self._unit = max(o.block_size, self.runner.reserve_unit())
        self.total_pages = o.context_tokens // self._unit
        self.free_credits = self.total_pages
        self.waiting: List[Request] = []
        self.active: List[Request] = []
        self.finished = {}
        self._next_id = 0
        self._order = 0
        self.failed = False
        self.stats = dict(batches=0, mixed_batches=0, prefill_tokens=0, decode_tokens=0, generated_tokens=0,
                          max_batch_tokens=0, max_batch_sequences=0, admission_waits=0, cancelled=0, timeouts=0)

    def warm_up(self, batch_sizes=None, contexts=None):
        """Captures the decoding steps ahead of the first requests (`Runner.warm_up`); to be called while the
        engine is idle.  Returns the number of graphs captured."""
        if self.active:
            raise RuntimeError("warm_up: the engine has running requests")
        return self.runner.warm_up(batch_sizes, contexts)

    # -- submit ----------------------------------------------------------------------------------
    def submit(self, prompt, max_tokens=64, temperature=0.0, seed=None, ignore_eos=False, priority=0,
               timeout_ms=None):
        """Queues a request and returns its id.  `timeout_ms` (1 .. 300000, as the reference allows,
        src/engine.cpp:658): the request ends with the reason "timeout" at the first step boundary after
        that long, waiting or running, and keeps what it has generated."""
        o = self.options
        if self.failed:
            raise RuntimeError("the engine stopped (a failed step, or shut down)")
        prompt = [int(t) for t in prompt]
        vocab = self.model.spec.vocab_size
        if not prompt:
            raise ValueError("empty prompt")
        if any(t < 0 or t >= vocab for t in prompt):
            raise ValueError("prompt holds a token id outside the vocabulary")
        if max_tokens < 1:
            raise ValueError("max_tokens must be at least 1")
        if len(prompt) + max_tokens > o.max_model_len:
            raise ValueError("prompt + max_tokens exceed max_model_len")
        if self._pages_for(len(prompt) + max_tokens) > self.total_pages:
            raise ValueError("the request does not fit an otherwise idle page pool")
        if not 0 <= priority <= 3:
            raise ValueError("priority must be in 0..3")
        if temperature < 0:
            raise ValueError("temperature must not be negative")
        if timeout_ms is not None and not 1 <= timeout_ms <= 300000:
            raise ValueError("timeout_ms must be in 1..300000")
        if len(self.waiting) >= o.queue_capacity:
            raise RuntimeError("the waiting queue is full")
        now = self.clock()
        rid = self._next_id
        self._next_id += 1
        req = Request(rid, prompt, max_tokens, float(temperature), rid if seed is None else int(seed),
                      bool(ignore_eos), priority, order=self._order, created=now, last_scheduled=now)
        req.rng = RequestRng(req.seed)
        req.deadline = None if timeout_ms is None else now + timeout_ms / 1000.0
        self._order += 1
        self.waiting.append(req)
        return rid

    def cancel(self, request_id):
        """Asks a waiting or running request to end; it does at the next step boundary, with the reason
        "cancelled" (src/engine.cpp:262-284, 709-716).  False when no such request waits or runs."""
        for req in self.waiting + self.active:
            if req.id == request_id:
                req.cancelled = True
                return True
        return False

    def shutdown(self):
        """Ends every waiting and running request with the reason "cancelled" and takes no new ones
        (src/engine.cpp:637).  Returns the events."""
        for req in self.waiting + self.active:
            req.cancelled = True
        events = self.expire()
        self.failed = True
        return events

    def expire(self):
        """Ends what was cancelled or has run out of time (every `step` begins with it, before the next batch
        is formed): a waiting request leaves the queue, a running one gives back its slot, its pages and its
        reservation.  Returns the events."""
        now = self.clock()
        events = []
        for req in [r for r in self.waiting + self.active if r.cancelled or (r.deadline is not None and now >= r.deadline)]:
            reason = "cancelled" if req.cancelled else "timeout"
            self.stats["cancelled" if req.cancelled else "timeouts"] += 1
            if req.slot is None:
                self.waiting.remove(req)
                req.finish_reason = reason
                self.finished[req.id] = req
            else:
                self._finish(req, reason)
            events.append((req.id, None, reason))
        return events

    def _pages_for(self, tokens):
        return (tokens + self._unit - 1) // self._unit

    # -- admission -------------------------------------------------------------------------------
    def _admit_waiting(self):
        """The decision is `admit`'s (native, a pure function of the queue); here it is carried out: a slot and
        the pages of its whole life for every request that starts, the queue left in the order of the walk."""
        if not self.waiting:
            return
        o = self.options
        now = self.clock()
        items = [(self._pages_for(len(r.prompt) + r.max_tokens), r.priority, int((now - r.created) * 1000), r.order)
                 for r in self.waiting]
        walk, started, waits = admit(items, self.free_credits, self.runner.free_slots(), o.aging_ms,
                                     o.admission_reserve_ms)
        self.stats["admission_waits"] += waits
        queue = [self.waiting[i] for i in walk]
        for i in started:
            req = self.waiting[i]
            req.slot = self.runner.open_request()
            req.pages = items[i][0]
            self.free_credits -= req.pages
            self.active.append(req)
        going = set(started)
        self.waiting = [r for i, r in zip(walk, queue) if i not in going]

    def _finish(self, req, reason):
        req.finish_reason = reason
        self.runner.close_request(req.slot)
        self.free_credits += req.pages
        req.slot, req.pages = None, 0
        self.active.remove(req)
        self.finished[req.id] = req

    # -- one iteration ---------------------------------------------------------------------------
    def step(self):
        """End what was cancelled or timed out, admit, form one batch, run it, sample, finish.  Returns the
        events of this iteration: [(request id, token or None, finish reason or None)]."""
        if self.failed:
            raise RuntimeError("the engine stopped after a failed step")
        o = self.options
        expired = self.expire()
        self._admit_waiting()
        if not self.active:
            if self.waiting:
                raise RuntimeError("no request fits an otherwise idle KV pool")
            return expired
        now = self.clock()
        items = [(i, len(r.prompt) - r.processed, r.priority, int((now - r.last_scheduled) * 1000), r.order)
                 for i, r in enumerate(self.active)]
        slices = schedule_batch(items, o.batch_tokens, o.prefill_chunk, o.policy, o.aging_ms, o.portion_step)
        if not slices:
            raise RuntimeError("scheduler made no progress")
        entries, sampled = [], []
        prefill_tokens = decode_tokens = 0
        for key, count, is_prefill in slices:
            req = self.active[key]
            if is_prefill:
                tokens = req.prompt[req.processed:req.processed + count]
                last = req.processed + count == len(req.prompt)
                entries.append(Entry(req.slot, tokens, [count - 1] if last else []))
                if last:
                    sampled.append(req)
                prefill_tokens += count
            else:
                entries.append(Entry(req.slot, [req.generated[-1]], [0]))
                sampled.append(req)
                decode_tokens += 1
        try:
            logits = self.runner.step(entries)
            tokens = []
            if sampled:
                tokens = self.sampler.sample(logits, [r.temperature for r in sampled],
                                             [r.rng.uniform() if r.temperature > 0 else 0.0 for r in sampled])
            vocab = self.model.spec.vocab_size
            if len(tokens) != len(sampled) or any(t < 0 or t >= vocab for t in tokens):
                raise RuntimeError("the step returned an invalid sample")
        except Exception:
            self.failed = True            # nothing of this batch is published
            raise
        s = self.stats
        s["batches"] += 1
        s["mixed_batches"] += int(prefill_tokens > 0 and decode_tokens > 0)
        s["prefill_tokens"] += prefill_tokens
        s["decode_tokens"] += decode_tokens
        s["max_batch_tokens"] = max(s["max_batch_tokens"], prefill_tokens + decode_tokens)
        s["max_batch_sequences"] = max(s["max_batch_sequences"], len(slices))
        done_at = self.clock()
        for key, count, is_prefill in slices:
            req = self.active[key]
            req.last_scheduled = done_at
            if is_prefill:
                req.processed += count
        events = []
        eos = set(self.model.spec.eos_token_ids)
        for req, token in zip(sampled, tokens):
            req.generated.append(token)
            s["generated_tokens"] += 1
            reason = None
            if token in eos and not req.ignore_eos:
                reason = "stop"
            elif len(req.generated) >= req.max_tokens:
                reason = "length"
            events.append((req.id, token, reason))
        for rid, _, reason in events:
            if reason is not None:
                self._finish(next(r for r in self.active if r.id == rid), reason)
        return expired + events

    def has_work(self):
        return bool(self.waiting or self.active)

    def run_until_done(self):
        """Drive steps until nothing waits or runs; {request id: generated tokens}."""
        while self.has_work():
            self.step()
        return {rid: list(r.generated) for rid, r in self.finished.items()}
