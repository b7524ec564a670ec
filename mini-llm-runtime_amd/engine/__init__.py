from .context import StepContext, Workspace
from .step import Entry, Runner, StepError

__all__ = ["StepContext", "Workspace", "Entry", "Runner", "StepError"]
