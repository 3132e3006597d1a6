from .context import Lane, StepContext, build_step_context
from .engine import Engine, StepError, resolve_dtype
from .model import DecoderModel

__all__ = ["DecoderModel", "Engine", "Lane", "StepContext", "StepError", "build_step_context", "resolve_dtype"]
