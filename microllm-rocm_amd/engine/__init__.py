from .batch import StepContext, StepEntry
from .engine import Engine, parse_dtype

__all__ = ["Engine", "StepContext", "StepEntry", "parse_dtype"]
