"""The engine: step function, scheduler, request loop."""
from .batch import StepContext, StepEntry, build_step
from .runner import ModelRunner, load_model, parse_dtype, random_model

__all__ = ["ModelRunner", "StepContext", "StepEntry", "build_step", "load_model", "parse_dtype",
           "random_model"]
from .engine import Completion, Engine, EngineStats  # noqa: E402
from .scheduler import Schedule, Scheduler  # noqa: E402

__all__ += ["Completion", "Engine", "EngineStats", "Schedule", "Scheduler"]
