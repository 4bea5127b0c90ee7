from .context import StepContext, StepEntry, build_context
from .engine import Engine
from .model import Model, build_parts
from .runner import ModelRunner
from .scheduler import PlannedEntry, Request, Scheduler

__all__ = ["Engine", "Model", "ModelRunner", "PlannedEntry", "Request", "Scheduler", "StepContext", "StepEntry",
           "build_context", "build_parts"]
