from .context import StepContext, Uploader, Workspace
from .scheduler import Engine, EngineOptions, Request, effective_priority, schedule_batch
from .step import Entry, Runner, StepError

__all__ = ["StepContext", "Workspace", "Engine", "EngineOptions", "Request", "effective_priority",
           "schedule_batch", "Entry", "Runner", "StepError"]
