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
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Tuple

import torch

from .safetensors_io import SafetensorsError, SafetensorsFile


class WeightError(ValueError):
    pass


@dataclass(frozen=True)
class WeightSpec:
    shape: Tuple[int, ...]
    keep_float32: bool = False     # norm weights and other small 32-bit vectors
    optional: bool = False         # e.g. lm_head of a tied model


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


def load_weights(folder, expected, dtype, device):
    """Return {name: device tensor} for every expected tensor that the folder holds."""
    names, files = open_model_folder(folder)
    try:
        check_names(expected, {n: f.entries[n] for n, f in names.items()})
        out = {}
        for name, spec in expected.items():
            if name not in names:
                continue
            t = names[name].tensor(name)
            if t.dtype.is_floating_point:
                if not torch.isfinite(t.float() if t.dtype != torch.float64 else t).all():
                    raise WeightError(f"tensor {name} holds values that are not finite")
                target = torch.float32 if (spec.keep_float32 or dtype == torch.float32) else dtype
                out[name] = t.to(device=device, dtype=target, copy=True).contiguous()
            elif t.dtype == torch.bool:
                raise WeightError(f"tensor {name}: boolean tensors are not supported")
            else:
                out[name] = t.to(device=device, dtype=torch.int32, copy=True).contiguous()
        return out
    finally:
        for f in files:
            f.close()
