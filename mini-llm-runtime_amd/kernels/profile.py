"""Time per kernel class inside the program: a pair of events around every launch, summed by class.

The reference records per-stage times inside its runtime (src/minillm/runtime.cpp:26-57,
include/minillm/profile.h:11-31; device time src/minillm/cuda/runtime.cpp:176,215,225-230).  Here a
`Profiler` attached to a `Kernels` object (`Kernels.profiler`) brackets each launch with two events on
the launch's stream; a profiled runner runs every step eagerly, since events inside a captured graph
measure nothing.  Classes: embed, norm, gemm (every projection, fused norm and activation
included), rope_kv, attention (merge of key splits included), activation, sampler, check.  With the
bytes a launch has to move and the flops it has to do (from its operands' shapes; for attention from
the step's contexts), the report gives GB/s and TFLOP/s per class.
"""
from __future__ import annotations

import functools

import torch

CLASSES = ("embed", "norm", "gemm", "rope_kv", "attention", "activation", "sampler", "check")


class Profiler:
    def __init__(self):
        self._open = []            # (class, start event, end event, bytes, flops) not yet read
        self._sums = {}            # class -> [calls, ms, bytes, flops]
        self._pending = None       # work stated by a part for the launch that follows
        self._pool = []

    def _event(self):
        return self._pool.pop() if self._pool else torch.cuda.Event(enable_timing=True)

    def next_work(self, nbytes, flops):
        """Bytes and flops of the next launch, for launches whose operands do not tell (attention)."""
        self._pending = (nbytes, flops)

    def start(self, kind, nbytes, flops):
        if self._pending is not None and nbytes == 0 and flops == 0:
            nbytes, flops = self._pending
        self._pending = None
        start, end = self._event(), self._event()
        start.record()
        return (kind, start, end, nbytes, flops)

    def stop(self, token):
        token[2].record()
        self._open.append(token)
        if len(self._open) >= 4096:
            self.collect()

    def collect(self):
        if self._open:
            self._open[-1][2].synchronize()
        for kind, start, end, nbytes, flops in self._open:
            entry = self._sums.setdefault(kind, [0, 0.0, 0, 0])
            entry[0] += 1
            entry[1] += start.elapsed_time(end)
            entry[2] += nbytes
            entry[3] += flops
            self._pool += [start, end]
        self._open = []

    def reset(self):
        self.collect()
        self._sums = {}

    def report(self):
        """{class: {calls, ms, gb_s, tflop_s}} and "total_ms", over everything since the last reset."""
        self.collect()
        out = {}
        for kind in CLASSES:
            if kind in self._sums:
                calls, ms, nbytes, flops = self._sums[kind]
                seconds = ms / 1e3
                out[kind] = {"calls": calls, "ms": round(ms, 4),
                             "gb_s": _significant(nbytes / seconds / 1e9) if seconds > 0 else None,
                             "tflop_s": _significant(flops / seconds / 1e12) if seconds > 0 else None}
        out["total_ms"] = round(sum(v[1] for v in self._sums.values()), 4)
        return out


def _significant(value, digits=4):
    """`value` to `digits` significant digits: a small model's rates (a first product's time holds the
    library's set-up) stay above zero where a fixed number of decimals would round them away."""
    return float(f"{value:.{digits}g}")


def timed(kind, work=None):
    """Decorator for a method of `Kernels`: with a profiler attached, the launch is bracketed by events.
    `work(self, *args, **kwargs)` returns (bytes, flops) of the launch."""
    def wrap(fn):
        @functools.wraps(fn)
        def inner(self, *args, **kwargs):
            profiler = self.profiler
            if profiler is None:
                return fn(self, *args, **kwargs)
            nbytes, flops = work(self, *args, **kwargs) if work is not None else (0, 0)
            token = profiler.start(kind, nbytes, flops)
            try:
                return fn(self, *args, **kwargs)
            finally:
                profiler.stop(token)
        return inner
    return wrap
