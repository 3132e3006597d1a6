from .context import Lane, PackedLanes, StepContext, StepTable, build_step_context
from .engine import Engine, StepError, StepFailed, resolve_dtype
from .generate import LLM, GenerationResult, generate
from .model import DecoderModel
from .scheduler import EngineConfig, QueueFull, Request, Scheduler

__all__ = ["DecoderModel", "Engine", "EngineConfig", "GenerationResult", "LLM", "Lane", "PackedLanes", "QueueFull",
           "Request", "Scheduler", "StepContext", "StepError", "StepFailed", "StepTable", "build_step_context", "generate", "resolve_dtype"]
