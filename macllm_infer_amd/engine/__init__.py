from .context import Lane, StepContext, build_step_context
from .engine import Engine, StepError, StepFailed, resolve_dtype
from .generate import LLM, GenerationResult, generate
from .model import DecoderModel
from .scheduler import EngineConfig, QueueFull, Request, Scheduler

__all__ = ["DecoderModel", "Engine", "EngineConfig", "GenerationResult", "LLM", "Lane", "QueueFull", "Request",
           "Scheduler", "StepContext", "StepError", "StepFailed", "build_step_context", "generate", "resolve_dtype"]
