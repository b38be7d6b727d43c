from .batch import StepContext, StepEntry, build_context
from .loading import build_model, get_ops, load_model, parse_dtype, random_model
from .runner import ModelRunner
from .scheduler import Request, Scheduler, SchedulerConfig, StepPlan
from .engine import Engine

__all__ = ["StepContext", "StepEntry", "build_context", "build_model", "get_ops", "load_model", "parse_dtype",
           "random_model", "ModelRunner", "Request", "Scheduler", "SchedulerConfig", "StepPlan", "Engine"]
