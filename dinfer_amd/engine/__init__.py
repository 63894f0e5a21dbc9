from .batch import Entry, StepBatch
from .request import Request
from .scheduler import Scheduler, SchedulerOutput

__all__ = ["Entry", "StepBatch", "Request", "Scheduler", "SchedulerOutput"]
