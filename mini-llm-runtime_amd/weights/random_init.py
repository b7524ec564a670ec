"""Random-weights mode: write a model folder (config.json, model.safetensors) from a
configuration and a seed.  Matrices are N(0, 0.02), norm weights 1 + N(0, 0.1); every tensor
has a generator of its own, seeded from (seed, tensor name), so the values of one tensor do
not depend on which other tensors exist."""
from __future__ import annotations

import hashlib
import json
import os

import torch

from .safetensors_io import write_safetensors


def _generator(seed, name):
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    g = torch.Generator(device="cpu")
    g.manual_seed(int.from_bytes(digest[:8], "little") & 0x7FFFFFFFFFFFFFFF)
    return g


def random_tensors(expected, seed, dtype=torch.bfloat16, matrix_std=0.02, norm_std=0.1):
    """expected: {name: WeightSpec}.  Optional tensors are left out.  Every tensor has a generator of its own,
    so they are drawn side by side in threads (the values do not depend on how many)."""
    from concurrent.futures import ThreadPoolExecutor

    def draw(item):
        name, spec = item
        g = _generator(seed, name)
        if spec.keep_float32:
            t = 1.0 + norm_std * torch.randn(spec.shape, generator=g, dtype=torch.float32)
        else:
            t = matrix_std * torch.randn(spec.shape, generator=g, dtype=torch.float32)
        return name, t.to(dtype)
    todo = [(name, spec) for name, spec in expected.items() if not spec.optional]
    workers = max(1, min(16, os.cpu_count() or 1, len(todo)))
    if workers == 1 or sum(_numel(spec.shape) for _, spec in todo) < (1 << 22):
        return dict(draw(item) for item in todo)
    with ThreadPoolExecutor(max_workers=workers) as pool:
        return dict(pool.map(draw, todo))              # (in the order of `expected`)


def _numel(shape):
    count = 1
    for extent in shape:
        count *= int(extent)
    return count


def write_random_model(folder, config, seed, dtype=torch.bfloat16, matrix_std=0.02, norm_std=0.1):
    """`config` is an architecture's configuration object (e.g. Qwen3Config)."""
    from ..parts.model import expected_tensors

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config.to_dict(), f, indent=1)
    expected = expected_tensors(config)
    tensors = random_tensors(expected, seed, dtype, matrix_std, norm_std)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors,
                      {"format": "pt", "seed": seed})
    return folder
