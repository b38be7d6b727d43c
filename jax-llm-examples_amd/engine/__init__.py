from .batch import StepContext, StepEntry, build_context
from .loading import build_model, get_ops, load_model, parse_dtype, random_model
from .runner import ModelRunner

__all__ = ["StepContext", "StepEntry", "build_context", "build_model", "get_ops", "load_model", "parse_dtype",
           "random_model", "ModelRunner"]
