"""Token choice: greedy (largest logit, ties -> lowest id, as the reference's argmax kernel,
src/minillm/cuda/ops.cu:166-201) and temperature sampling (p = softmax(logits / T), inverse-CDF
draw).  The reference serves greedy only (src/http_server.cpp:140-142); temperature is this
engine's addition.

The uniform number of a draw comes from the request's own generator state (seed, number of
draws so far), never from a shared stream: which token a request gets does not depend on the
other requests of the batch.  A row of logits that holds a NaN or an infinity is an error.
"""
from __future__ import annotations

import torch

_MASK = (1 << 64) - 1


def splitmix64(x):
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    z = x
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


class RequestRng:
    """Counter-based generator: the n-th draw of a request is a pure function of (seed, n)."""

    def __init__(self, seed):
        self.seed = int(seed) & _MASK
        self.draws = 0

    def uniform(self):
        """A float in [0, 1) with 24 random bits (exact in 32-bit)."""
        z = splitmix64(splitmix64(self.seed) ^ ((self.draws * 0xD1342543DE82EF95) & _MASK))
        self.draws += 1
        return (z >> 40) / float(1 << 24)


class NonFiniteLogits(RuntimeError):
    pass


class Sampler:
    def __init__(self, kernels, device, max_rows=64):
        self.kernels = kernels
        self.device = torch.device(device)
        kernels.prepare(["sampling"])
        self._grow(max_rows)

    def _grow(self, rows):
        self.max_rows = rows
        self._params = torch.empty((2, rows), dtype=torch.float32, device=self.device)
        self._host = torch.empty((2, rows), dtype=torch.float32).pin_memory()
        self._tokens = torch.empty(rows, dtype=torch.int32, device=self.device)
        self._status = torch.zeros(2, dtype=torch.int32, device=self.device)
        need_f, need_i = self.kernels.sample_scratch(rows)
        self._scratch_f = torch.empty(need_f, dtype=torch.float32, device=self.device)
        self._scratch_i = torch.empty(need_i, dtype=torch.int32, device=self.device)

    def sample(self, logits, temperatures, uniforms):
        """logits: float [R, V] on the device; per row a temperature (<= 0: greedy) and a uniform
        number.  Returns R token ids."""
        rows = logits.shape[0]
        if len(temperatures) != rows or len(uniforms) != rows:
            raise ValueError("one temperature and one uniform number per row")
        if rows > self.max_rows:
            self._grow(max(rows, 2 * self.max_rows))
        self._host[0, :rows] = torch.tensor(temperatures, dtype=torch.float32)
        self._host[1, :rows] = torch.tensor(uniforms, dtype=torch.float32)
        self._params[:, :rows].copy_(self._host[:, :rows], non_blocking=True)
        temp = self._params[0, :rows]
        uni = self._params[1, :rows]
        tokens = self._tokens[:rows]
        self.kernels.sample(logits, temp, uni, tokens, self._status, self._scratch_f, self._scratch_i,
                            any_sampling=any(t > 0 for t in temperatures))
        out = torch.cat([tokens, self._status]).cpu().tolist()     # one copy back, one sync
        if out[rows] != 0:
            raise NonFiniteLogits(f"row {out[rows + 1]} of the logits holds a value that is not finite")
        return out[:rows]
