"""Rotary position encoding over the whole head, split-half pairing (j, j + dim/2):
freq_j = base^(-2j/dim), angle = position * freq_j held in 32-bit, as the reference computes it
(src/minillm/runtime.cpp:231-241, table form src/minillm/cuda/storage.cpp:261-287).  The table
[max_positions, dim] holds cos in its first half and sin in its second.  The part hands the attention
part a `Rotation`: this table, the rotated width (here the whole head) and the pairing (here split-half)."""
from __future__ import annotations

import numpy as np
import torch

from .registry import Rotation, register_part


@register_part("position", "rope_split_half")
class RopeSplitHalf:
    def __init__(self, spec):
        self.dim, self.base = spec.dim, float(spec.base)
        self._tables = {}

    def rotation(self, max_positions, device):
        """The whole head in split-half pairs."""
        return Rotation(self.rotation_table(max_positions, device), self.dim, interleaved=False)

    def rotation_table(self, max_positions, device):
        key = (max_positions, str(device))
        if key not in self._tables:
            half = self.dim // 2
            j = np.arange(half, dtype=np.float64)
            freq = np.power(self.base, -2.0 * j / self.dim).astype(np.float32)
            angle = (np.arange(max_positions, dtype=np.float32)[:, None] * freq[None, :]).astype(np.float32)
            table = np.concatenate([np.cos(angle.astype(np.float64)), np.sin(angle.astype(np.float64))],
                                   axis=1).astype(np.float32)
            self._tables[key] = torch.from_numpy(table).to(device)
        return self._tables[key]
