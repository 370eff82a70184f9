from .batch import StepContext, StepEntry
from .engine import Engine, StepError, parse_dtype
from .model import Model, expected_params_of_spec
from .scheduler import Request, Scheduler

__all__ = ["StepContext", "StepEntry", "Engine", "StepError", "parse_dtype", "Model",
           "expected_params_of_spec", "Request", "Scheduler"]
