"""The engine: step function, scheduler and generation."""

from .batch import EntryView, StepEntry, StepError, StepState, check_entries
from .engine import Engine, resolve_dtype
from .model import BuiltModel
from .scheduler import PlannedEntry, Request, Scheduler, SchedulerError

__all__ = ["Engine", "StepEntry", "StepError", "EntryView", "StepState", "BuiltModel", "resolve_dtype", "PlannedEntry", "Request",
           "Scheduler", "SchedulerError"]
