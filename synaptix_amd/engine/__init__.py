from .batch import StepLayout, StepContext
from .engine import Engine, StepError, parse_dtype

__all__ = ["StepLayout", "StepContext", "Engine", "StepError", "parse_dtype"]
