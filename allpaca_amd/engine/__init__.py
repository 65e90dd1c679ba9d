from .batch import Entry, StepInfo
from .engine import Engine
from .runner import ModelRunner, StepError
from .scheduler import Plan, Request, RequestTooLarge, Scheduled, Scheduler

__all__ = ["Entry", "StepInfo", "Engine", "ModelRunner", "StepError", "Plan", "Request", "RequestTooLarge",
           "Scheduled", "Scheduler"]
