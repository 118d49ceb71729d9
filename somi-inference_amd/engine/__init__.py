"""Step function, scheduler and the generation loop."""

from .batch import EntryInfo, PagedView, StepBatch, StepEntry, build_step
from .runner import ModelRunner, StepError

__all__ = ["EntryInfo", "ModelRunner", "PagedView", "StepBatch", "StepEntry", "StepError", "build_step"]
