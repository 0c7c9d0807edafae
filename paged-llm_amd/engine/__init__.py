from .batch import StepContext, StepEntry
from .request import EndReason, Request, SamplingParams, Stage
from .scheduler import Grant, Scheduler, StepPlan

__all__ = ["StepContext", "StepEntry", "Request", "Stage", "EndReason", "SamplingParams", "Grant", "Scheduler", "StepPlan"]
