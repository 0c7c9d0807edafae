from .batch import StepContext, StepEntry
from .request import Request, RequestStatus, SamplingParams
from .scheduler import ScheduledRequest, Scheduler, SchedulerOutput

__all__ = ["StepContext", "StepEntry", "Request", "RequestStatus", "SamplingParams", "ScheduledRequest", "Scheduler",
           "SchedulerOutput"]
