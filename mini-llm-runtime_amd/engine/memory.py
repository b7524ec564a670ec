"""The device memory a runner will hold, computed before anything is allocated.

The reference computes the plan of its arenas first, compares it with the budget
min(the user's cap, 80 % of free memory, free - 512 MiB), allocates, and asserts that what was
allocated is what was planned (src/minillm/cuda/storage.cpp:44-181, src/minillm/cuda/runtime.cpp:134).
Here the weights have their own planned arena (weights/loader.py, gated when the model is loaded);
this module plans the rest: the cache (pages, block tables, state of fixed size), the scratch
buffers that the parts name for the largest step (`workspace_plan`), the logits, the step's
metadata and the vendor library's scratch.  `Runner` checks the plan against the budget before
the cache is allocated, and `Runner.memory_report` shows plan beside actual."""
from __future__ import annotations

from dataclasses import asdict, dataclass

import torch

from ..weights.loader import MemoryBudgetError, device_budget

__all__ = ["MemoryBudgetError", "MemoryPlan", "device_budget", "element_size"]


def element_size(dtype):
    return torch.empty((), dtype=dtype).element_size()


@dataclass
class MemoryPlan:
    weights: int = 0              # already resident when a runner is built
    kv_pages: int = 0
    block_tables: int = 0
    state: int = 0
    workspace: int = 0            # the parts' scratch buffers at the largest step, logits included
    metadata: int = 0
    library_scratch: int = 0

    def to_allocate(self):
        """What building the runner and running its largest step will allocate."""
        return self.kv_pages + self.block_tables + self.state + self.workspace + self.metadata + self.library_scratch

    def total(self):
        return self.weights + self.to_allocate()

    def as_dict(self):
        return {**asdict(self), "total": self.total()}

    def check(self, user_cap, device):
        """Raises MemoryBudgetError when the plan does not fit; `user_cap` None: no gate, 0: no cap of the
        user's, only the rule's share of the free memory."""
        if user_cap is None or torch.device(device).type != "cuda":
            return
        budget = device_budget(user_cap, device)
        if self.to_allocate() > budget:
            parts = ", ".join(f"{k} {v}" for k, v in self.as_dict().items() if k not in ("weights", "total") and v)
            raise MemoryBudgetError(f"the runner needs {self.to_allocate()} bytes of device memory ({parts}) beside "
                                    f"{self.weights} bytes of weights and exceeds the budget of {budget} bytes")
