"""Weights by tensor name.

`open_model_folder` finds the safetensors files of a model folder (one `model.safetensors`,
or the shards that `model.safetensors.index.json` names).  `load_weights` compares what the
model expects ({name: WeightSpec}) with what the files hold and raises ONE error that lists
every missing tensor, every unexpected tensor and every wrong shape, the way the reference
refuses a file tensor by tensor (src/minillm/qwen3_model.cpp:42-49,
src/minillm/gguf_model.cpp:182-187).  Then it copies the tensors to the device:

  * matrices and tables of floating type are kept in bfloat16 for the bfloat16 engine
    (a matrix stored in 32-bit is rounded once, at load) and widened to float32 for the
    float32 engine;
  * vectors marked `keep_float32` (norm weights) are float32 in both engines: the norms are
    computed in 32-bit;
  * integer tables become int32.

Device memory is planned before anything is allocated: from the expected tensors and what the
files hold, every tensor gets an offset in ONE arena (offsets are multiples of 256 bytes), the
total is compared with the budget (`MemoryBudgetError` when it does not fit, nothing allocated),
then the arena is allocated once and every tensor is copied to its place.  Tensors whose specs
carry the same `stack` name lie one after the other, row block after row block, so that a part
can use them as one matrix without a second copy (`stacked`).  The reference plans its weight
arena the same way (src/minillm/cuda/storage.cpp:44-152) and asserts actual == planned
(src/minillm/cuda/runtime.cpp:134); here `WeightArena.used == WeightArena.planned` by construction
and is asserted after the upload.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from .safetensors_io import SafetensorsError, SafetensorsFile


class WeightError(ValueError):
    pass


class MemoryBudgetError(RuntimeError):
    """What is about to be allocated does not fit the device budget; nothing was allocated."""


@dataclass(frozen=True)
class WeightSpec:
    shape: Tuple[int, ...]
    keep_float32: bool = False     # norm weights and other small 32-bit vectors
    optional: bool = False         # e.g. lm_head of a tied model
    stack: Optional[str] = None    # matrices of equal width with the same name here lie row block after
                                   # row block in memory, in the order of their specs (see `stacked`)


ALIGN = 256


def device_budget(user_cap, device):
    """Bytes that may still be allocated on `device`: the reference's rule
    min(the user's cap, 80 % of what is free, what is free - 512 MiB) (src/minillm/cuda/storage.cpp:168-175),
    a cap of 0 meaning none."""
    free, _ = torch.cuda.mem_get_info(device)
    limit = min(int(free * 0.8), free - (512 << 20))
    return min(limit, user_cap) if user_cap else limit


def _target_dtype(found_dtype, spec, dtype):
    if found_dtype.is_floating_point:
        return torch.float32 if (spec.keep_float32 or dtype == torch.float32) else dtype
    return torch.int32


def plan_arena(expected, found, dtype):
    """expected: {name: WeightSpec} in the model's order; found: {name: (dtype, shape)} of the files.
    Returns ([(offset, [names], target dtype)], total bytes): one allocation per tensor, or per run of
    neighbours that share a `stack` name."""
    allocations, at = [], 0
    names = [n for n in expected if n in found]
    i = 0
    while i < len(names):
        spec = expected[names[i]]
        target = _target_dtype(found[names[i]][0], spec, dtype)
        group = [names[i]]
        if spec.stack is not None and len(spec.shape) == 2:
            while i + len(group) < len(names):
                nxt = expected[names[i + len(group)]]
                if nxt.stack != spec.stack or len(nxt.shape) != 2 or nxt.shape[1] != spec.shape[1] or \
                        _target_dtype(found[names[i + len(group)]][0], nxt, dtype) != target:
                    break
                group.append(names[i + len(group)])
        size = sum(_numel(expected[n].shape) for n in group) * torch.empty((), dtype=target).element_size()
        allocations.append((at, group, target))
        at += -(-size // ALIGN) * ALIGN
        i += len(group)
    return allocations, at


def _numel(shape):
    count = 1
    for extent in shape:
        count *= int(extent)
    return count


class WeightArena:
    """One device allocation that holds every tensor of a model at its planned offset."""

    def __init__(self, planned, device):
        self.planned = planned
        self.used = 0
        self.memory = torch.empty(max(planned, 1), dtype=torch.uint8, device=device)

    def place(self, offset, shape, dtype):
        size = _numel(shape) * torch.empty((), dtype=dtype).element_size()
        self.used = max(self.used, -(-(offset + size) // ALIGN) * ALIGN)
        if offset + size > self.memory.numel():
            raise WeightError("a tensor does not fit its planned place")       # the plan is wrong
        return self.memory[offset:offset + size].view(dtype).view(shape)


def stacked(tensors):
    """One matrix [sum of rows, width] of the given matrices: without a copy where they lie one after
    the other in memory (as the loader places tensors that share a `stack` name), else a copy."""
    first = tensors[0]
    at = first.data_ptr()
    adjacent = all(t.is_contiguous() and t.dtype == first.dtype and t.shape[1:] == first.shape[1:] for t in tensors)
    for t in tensors:
        adjacent = adjacent and t.data_ptr() == at
        at += t.numel() * t.element_size()
    if adjacent and all(t.untyped_storage().data_ptr() == first.untyped_storage().data_ptr() for t in tensors):
        rows = sum(t.shape[0] for t in tensors)
        return torch.as_strided(first, (rows, *first.shape[1:]), first.stride())
    return torch.cat(tensors, dim=0).contiguous()


def open_model_folder(folder):
    """Return ({tensor name: file}, [files])."""
    index = os.path.join(folder, "model.safetensors.index.json")
    single = os.path.join(folder, "model.safetensors")
    names = {}
    files = []
    try:
        if os.path.isfile(index):
            with open(index) as f:
                weight_map = json.load(f)["weight_map"]
            opened = {}
            for tensor, shard in weight_map.items():
                if shard not in opened:
                    opened[shard] = SafetensorsFile(os.path.join(folder, shard))
                    files.append(opened[shard])
                if tensor not in opened[shard].entries:
                    raise WeightError(f"{index}: {tensor} is not in {shard}")
                names[tensor] = opened[shard]
        elif os.path.isfile(single):
            f = SafetensorsFile(single)
            files.append(f)
            names = {name: f for name in f.entries}
        else:
            raise WeightError(f"{folder}: no model.safetensors (or model.safetensors.index.json)")
    except SafetensorsError as err:
        raise WeightError(str(err)) from None
    return names, files


def check_names(expected, found):
    """expected: {name: WeightSpec}; found: {name: (dtype, shape)}.  Raises one WeightError
    naming everything that is wrong."""
    missing = sorted(n for n, s in expected.items() if n not in found and not s.optional)
    unexpected = sorted(n for n in found if n not in expected)
    wrong = []
    for name, spec in sorted(expected.items()):
        if name in found and tuple(found[name][1]) != tuple(spec.shape):
            wrong.append(f"{name}: expected {list(spec.shape)}, found {list(found[name][1])}")
    if missing or unexpected or wrong:
        parts = []
        if missing:
            parts.append(f"missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            parts.append(f"unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong:
            parts.append(f"wrong shapes ({len(wrong)}): " + "; ".join(wrong))
        raise WeightError("model weights do not match the configuration: " + " | ".join(parts))


def load_weights(folder, expected, dtype, device, device_budget_bytes=None, arena_out=None):
    """Return {name: device tensor} for every expected tensor that the folder holds.  The tensors are
    views of one arena, planned and checked against the budget before it is allocated.
    `device_budget_bytes`: None for no gate, else the user's cap (0: none) that enters the budget rule.
    `arena_out`: a list that receives the `WeightArena` (for reports and tests)."""
    names, files = open_model_folder(folder)
    try:
        found = {n: f.entries[n] for n, f in names.items()}
        check_names(expected, found)
        for name in expected:
            if name in found and found[name][0] == torch.bool:
                raise WeightError(f"tensor {name}: boolean tensors are not supported")
        allocations, total = plan_arena(expected, found, dtype)
        device = torch.device(device)
        if device_budget_bytes is not None and device.type == "cuda":
            budget = device_budget(device_budget_bytes, device)
            if total > budget:
                raise MemoryBudgetError(f"the weights need {total} bytes of device memory and exceed the budget of "
                                        f"{budget} bytes")
        arena = WeightArena(total, device)
        out = {}
        for offset, group, target in allocations:
            for name in group:
                spec = expected[name]
                t = names[name].tensor(name)
                if t.dtype.is_floating_point and \
                        not torch.isfinite(t.float() if t.dtype != torch.float64 else t).all():
                    raise WeightError(f"tensor {name} holds values that are not finite")
                place = arena.place(offset, spec.shape, target)
                place.copy_(t)
                out[name] = place
                offset += place.numel() * place.element_size()
        if arena.used != arena.planned:
            raise WeightError(f"the weight arena holds {arena.used} bytes where {arena.planned} were planned")
        if arena_out is not None:
            arena_out.append(arena)
        return out
    finally:
        for f in files:
            f.close()
