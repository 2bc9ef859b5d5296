from .batch import StepContext, StepEntry
from .engine import Engine, parse_dtype
from .generate import GenerationConfig, generate, generate_serial
from .scheduler import CompletionReason, Request, RequestState, Scheduler, SchedulerMetrics

__all__ = ["StepContext", "StepEntry", "Engine", "parse_dtype", "GenerationConfig", "generate", "generate_serial",
           "CompletionReason", "Request", "RequestState", "Scheduler", "SchedulerMetrics"]
