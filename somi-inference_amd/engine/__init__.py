"""Step function, scheduler and the generation loop."""

from .batch import EntryInfo, PagedView, StepBatch, StepEntry, build_step
from .engine import Engine
from .request import Request, RequestStatus
from .runner import ModelRunner, StepError
from .scheduler import ScheduledPortion, Scheduler, SchedulerError, SchedulerOutput

__all__ = ["Engine", "EntryInfo", "ModelRunner", "PagedView", "Request", "RequestStatus", "ScheduledPortion",
           "Scheduler", "SchedulerError", "SchedulerOutput", "StepBatch", "StepEntry", "StepError", "build_step"]
