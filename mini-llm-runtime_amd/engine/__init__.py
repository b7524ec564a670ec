from .context import StepContext, Uploader, Workspace
from .memory import MemoryBudgetError, MemoryPlan, device_budget
from .scheduler import Engine, EngineOptions, Request, admit, effective_priority, schedule_batch
from .step import Entry, NonFiniteHidden, Runner, StepError

__all__ = ["StepContext", "Workspace", "Engine", "EngineOptions", "Request", "admit", "effective_priority",
           "schedule_batch", "Entry", "Runner", "StepError", "NonFiniteHidden", "MemoryBudgetError", "MemoryPlan",
           "device_budget"]
