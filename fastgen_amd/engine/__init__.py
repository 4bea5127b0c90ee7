from .context import StepContext, StepEntry, build_context
from .model import Model, build_parts
from .runner import ModelRunner

__all__ = ["Model", "ModelRunner", "StepContext", "StepEntry", "build_context", "build_parts"]
