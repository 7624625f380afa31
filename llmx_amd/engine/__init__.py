"""The engine: step function, scheduler and generation."""

from .batch import EntryView, StepEntry, StepState
from .engine import Engine, StepError, resolve_dtype
from .model import BuiltModel
from .scheduler import PlannedEntry, Request, Scheduler, SchedulerError

__all__ = ["Engine", "StepEntry", "StepError", "EntryView", "StepState", "BuiltModel", "resolve_dtype", "PlannedEntry", "Request",
           "Scheduler", "SchedulerError"]
