from .step import StepEntry, StepError, StepFunction
from .loading import LoadedModel, load_model, parse_dtype
from .scheduler import PlanItem, Request, Scheduler, SchedulerError, StepPlan
from .engine import Engine

__all__ = ["StepEntry", "StepError", "StepFunction", "LoadedModel", "load_model", "parse_dtype", "PlanItem", "Request",
           "Scheduler", "SchedulerError", "StepPlan", "Engine"]
